"""GPU parity of f8f8bf16_rowwise against the dequantized-fp32 oracle (north_star tolerance:
max-rel 1e-2, normwise 2e-3) plus exact textbook cases.  Shapes follow the reference's tests
(test/gemm/gemm_test.py:204-213,354-506; test/gemm/triton/fp8_gemm_test.py:29-142)."""
import pytest
import torch

import mslk_amd
from mslk_amd import workloads as W
from oracle import c_twin
from oracle import fp8_rowwise_oracle as O
from tests.helpers import assert_gemm_close, assert_quant_bit_exact

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F8 = torch.float8_e4m3fn


def _quant_cpu(x):
    return O.quantize_fp8_row(x)


def _gpu(*ts):
    return [None if t is None else t.to(DEV) for t in ts]


def _op(xq, wq, xs, ws, bias=None):
    y = torch.ops.mslk.f8f8bf16_rowwise(*_gpu(xq, wq, xs, ws), bias=None if bias is None else bias.to(DEV))
    torch.cuda.synchronize()
    return y


def _random_problem(M, N, K, g, x_std=1.0, w_std=0.02):
    x = (torch.randn(M, K, generator=g) * x_std).bfloat16()
    w = (torch.randn(N, K, generator=g) * w_std).bfloat16()
    xq, xs = _quant_cpu(x)
    wq, ws = _quant_cpu(w)
    return xq, wq, xs, ws


SHAPES = [
    # (M, N, K): reference test shapes, tile edges, K tails, odd K, skinny M
    (256, 256, 128), (2048, 4096, 2048), (4096, 8192, 4096), (1024, 1024, 1024),
    (300, 520, 640), (257, 255, 384), (129, 1000, 4096), (512, 768, 144), (512, 512, 16), (384, 130, 2064),
    (100, 100, 100), (65, 33, 17), (70, 64, 1), (1, 8192, 8192), (4, 8192, 8192), (16, 8192, 8192), (64, 8192, 8192),
    (3, 1000, 272), (17, 260, 4096), (33, 48, 512), (48, 16, 128), (64, 15, 256), (1, 1, 16), (2, 7, 24),
    (300, 517, 256), (513, 1030, 384), (8, 100, 1024), (33, 48, 2048), (50, 1000, 3072), (64, 15, 1024), (5, 8200, 5120), (20, 513, 9216),
]


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_dense_matches_oracle(M, N, K):
    g = torch.Generator().manual_seed(M * 1315423911 % 2**31 + N * 31 + K)
    xq, wq, xs, ws = _random_problem(M, N, K, g)
    y = _op(xq, wq, xs, ws)
    assert y.shape == (M, N) and y.dtype == torch.bfloat16
    assert_gemm_close(y, O.dequant_matmul(xq, wq, xs, ws), f"{M}x{N}x{K}")


@pytest.mark.parametrize("M,N,K", [(512, 512, 256), (300, 260, 384), (16, 512, 512), (40, 300, 1040), (33, 20, 50)])
def test_exact_when_fp32_accumulation_is_exact(M, N, K):
    """Integer-valued codes in [-8, 8] and power-of-two scales: every partial sum is an integer below
    2^24, so the fp32 result is exact in any summation order and the bf16 output must match bit for bit."""
    g = torch.Generator().manual_seed(K)
    xi = torch.randint(-8, 9, (M, K), generator=g).float()
    wi = torch.randint(-8, 9, (N, K), generator=g).float()
    xq, wq = xi.to(F8), wi.to(F8)
    xs = 2.0 ** torch.randint(-3, 4, (M,), generator=g).float()
    ws = 2.0 ** torch.randint(-3, 4, (N,), generator=g).float()
    bias = torch.randint(-4, 5, (N,), generator=g).float()
    want = ((xi @ wi.T) * xs[:, None] * ws[None, :] + bias[None, :]).bfloat16()
    y = _op(xq, wq, xs, ws, bias)
    assert torch.equal(y.cpu(), want)
    small = c_twin.dequant_gemm(xq.view(torch.uint8)[:5], wq.view(torch.uint8)[:7], xs[:5], ws[:7], bias[:7])
    assert torch.equal(y.cpu()[:5, :7].double(), small.bfloat16().double())


@pytest.mark.parametrize("fp16_out", [False, True])
@pytest.mark.parametrize("bias_dtype", [None, torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(3072, 3328, 384), (4096, 4096, 128), (3072, 3072, 256), (3100, 3330, 640)])
def test_exact_on_full_256_tiles(M, N, K, bias_dtype, fp16_out):
    """129 ... 256 tiles of 256 x 256: without a bias, interior tiles run their last K step under the epilogue (K = 128
    is that step alone); the last shape adds ragged edge tiles, which take the ordinary epilogue, around them.  Exact
    arithmetic as above, so every output must match bit for bit."""
    g = torch.Generator().manual_seed(M + K)
    xi = torch.randint(-8, 9, (M, K), generator=g).float()
    wi = torch.randint(-8, 9, (N, K), generator=g).float()
    xs = 2.0 ** torch.randint(-3, 4, (M,), generator=g).float()
    ws = 2.0 ** torch.randint(-3, 4, (N,), generator=g).float()
    want = (xi @ wi.T) * xs[:, None] * ws[None, :]
    bias = None
    if bias_dtype is not None:
        bias = torch.randint(-4, 5, (N,), generator=g).float()
        want = want + bias[None, :]
        bias = bias.to(bias_dtype).to(DEV)
    op = torch.ops.mslk.f8f8f16_rowwise if fp16_out else torch.ops.mslk.f8f8bf16_rowwise
    y = op(*_gpu(xi.to(F8), wi.to(F8), xs, ws), bias=bias)
    torch.cuda.synchronize()
    assert torch.equal(y.cpu(), want.half() if fp16_out else want.bfloat16())


def test_measuring_build_of_the_tile_kernel_gives_the_product_bits_and_ordered_stamps():
    """mslk_amd_debug_gemm_phases is the 256 x 256 tile kernel with four counter readings per wave: it must write the very
    output of f8f8bf16_rowwise (exact integer arithmetic here), and every wave's readings must be in order."""
    import ctypes
    from mslk_amd import _lib
    M, N, K = 1024, 1280, 512
    g = torch.Generator().manual_seed(11)
    xi = torch.randint(-8, 9, (M, K), generator=g).float()
    wi = torch.randint(-8, 9, (N, K), generator=g).float()
    xs = 2.0 ** torch.randint(-3, 4, (M,), generator=g).float()
    ws = 2.0 ** torch.randint(-3, 4, (N,), generator=g).float()
    want = ((xi @ wi.T) * xs[:, None] * ws[None, :]).bfloat16()
    xq, wq, xsd, wsd = _gpu(xi.to(F8), wi.to(F8), xs, ws)
    tiles = (M // 256) * (N // 256)
    slots = (tiles + 7) // 8 * 8
    y = torch.zeros(M, N, dtype=torch.bfloat16, device=DEV)
    stamps = torch.zeros(slots * 16, dtype=torch.int64, device=DEV)
    L = _lib.lib()
    _lib.check(L.mslk_amd_debug_gemm_phases(xq.data_ptr(), wq.data_ptr(), xsd.data_ptr(), wsd.data_ptr(), y.data_ptr(), M, N, K,
                                            stamps.data_ptr(), torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert torch.equal(y.cpu(), want)
    assert torch.equal(y, torch.ops.mslk.f8f8bf16_rowwise(xq, wq, xsd, wsd))
    t = stamps.view(slots, 4, 4).cpu()
    written = t[..., 0] != 0
    assert int(written.all(dim=1).sum()) == tiles and int(written.any(dim=1).sum()) == tiles   # one workgroup per tile, all four waves
    w = t[written.all(dim=1)]
    assert bool((w[..., 0] <= w[..., 1]).all() and (w[..., 1] <= w[..., 2]).all() and (w[..., 2] <= w[..., 3]).all())
    assert int((w[..., 3] - w[..., 0]).max()) < 100_000   # 100 MHz counter: under a millisecond
    # shapes with edge tiles are refused: the measuring build has the interior path only
    assert L.mslk_amd_debug_gemm_phases(xq.data_ptr(), wq.data_ptr(), xsd.data_ptr(), wsd.data_ptr(), y.data_ptr(), M - 1, N, K,
                                        stamps.data_ptr(), None) != 0
    assert b"multiples of 256" in L.mslk_amd_last_error()


@pytest.mark.parametrize("tiles_m,tiles_n,K", [(2, 128, 1024), (1, 3, 128), (5, 7, 640)])
def test_operand_stream_probe_reads_its_operands_and_writes_nothing(tiles_m, tiles_n, K):
    """mslk_amd_debug_tile_streams issues the loads of the 128 x 64 tile kernel's K loop and nothing else: every variant
    runs to completion on operands of exactly the stated size (tile counts that do and do not fill the grid's multiple of
    8, K loops shorter and longer than the ring), and the operands and a guard region behind them are unchanged."""
    from mslk_amd import _lib
    g = torch.Generator().manual_seed(tiles_m * 100 + tiles_n)
    nx, nw = tiles_m * 128 * K, tiles_n * 64 * K
    buf = torch.randint(0, 255, (nx + nw + 4096,), dtype=torch.uint8, generator=g).to(DEV)
    before = buf.clone()
    L = _lib.lib()
    for which in (1, 2, 3):
        _lib.check(L.mslk_amd_debug_tile_streams(buf.data_ptr(), nx, buf.data_ptr() + nx, nw, K, tiles_m, tiles_n, which,
                                                 torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert torch.equal(buf, before)


def test_identity_and_one_hot_weights_select_dequantized_activations():
    g = torch.Generator().manual_seed(9)
    M, K = 300, 512
    x = torch.randn(M, K, generator=g).bfloat16()
    xq, xs = _quant_cpu(x)
    perm = torch.randperm(K, generator=g)
    w = torch.zeros(K, K)
    w[torch.arange(K), perm] = 1.0
    y = _op(xq, w.to(F8), xs, torch.ones(K))
    want = O.dequantize_fp8_row(xq, xs)[:, perm].bfloat16()
    assert torch.equal(y.cpu(), want)
    # all-ones codes: every output is K * xs[m] * ws[n]
    ones = torch.ones(64, 256).to(F8)
    xs1, ws1 = torch.rand(64, generator=g) + 0.5, torch.rand(64, generator=g) + 0.5
    y = _op(ones, ones, xs1, ws1)
    assert torch.equal(y.cpu(), ((256.0 * xs1)[:, None] * ws1[None, :]).bfloat16())


@pytest.mark.parametrize("bias_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(512, 768, 256), (16, 1024, 512), (100, 100, 100)])
def test_bias(bias_dtype, M, N, K):
    g = torch.Generator().manual_seed(21)
    xq, wq, xs, ws = _random_problem(M, N, K, g)
    bias = (torch.randn(N, generator=g) * 0.5).to(bias_dtype)
    y = _op(xq, wq, xs, ws, bias)
    assert_gemm_close(y, O.dequant_matmul(xq, wq, xs, ws, bias.float()), "bias")
    y0 = _op(xq, wq, xs, ws)
    shift = (y.float() - y0.float()).cpu()
    assert torch.allclose(shift, bias.float()[None, :].expand_as(shift), atol=2e-2, rtol=2e-2)


def test_out_variant_leading_dims_and_empty():
    g = torch.Generator().manual_seed(22)
    xq, wq, xs, ws = _random_problem(3 * 40, 384, 256, g)
    ref = O.dequant_matmul(xq, wq, xs, ws)
    xq3, xs3 = xq.view(3, 40, 256), xs.view(3, 40)
    y3 = _op(xq3, wq, xs3, ws)
    assert y3.shape == (3, 40, 384)
    assert_gemm_close(y3.reshape(120, 384), ref)
    out = torch.full((3, 40, 384), 7.0, dtype=torch.bfloat16, device=DEV)
    r = torch.ops.mslk.f8f8bf16_rowwise_out(*_gpu(xq3, wq, xs3, ws), out)
    torch.cuda.synchronize()
    assert r is None and torch.equal(out, y3)
    # empty inputs give zeros of the output shape (reference test shape (0, 256, 4096) and K == 0)
    e = torch.ops.mslk.f8f8bf16_rowwise(torch.empty(0, 256, dtype=F8, device=DEV), torch.zeros(4096, 256, device=DEV).to(F8),
                                        torch.empty(0, device=DEV), torch.ones(4096, device=DEV))
    assert e.shape == (0, 4096)
    z = torch.ops.mslk.f8f8bf16_rowwise(torch.empty(5, 0, dtype=F8, device=DEV), torch.empty(9, 0, dtype=F8, device=DEV),
                                        torch.ones(5, device=DEV), torch.ones(9, device=DEV))
    assert z.shape == (5, 9) and (z == 0).all()
    with pytest.raises(RuntimeError, match="use_fast_accum"):
        torch.ops.mslk.f8f8bf16_rowwise(*_gpu(xq, wq, xs, ws), use_fast_accum=False)
    with pytest.raises(RuntimeError, match="Scales must be float32"):
        torch.ops.mslk.f8f8bf16_rowwise(*_gpu(xq, wq, xs.half(), ws))


def test_unaligned_views_are_copied_or_take_the_generic_path():
    from mslk_amd import _lib
    g = torch.Generator().manual_seed(23)
    for (M, N, K) in [(40, 72, 96), (300, 1030, 1024)]:
        xq, wq, xs, ws = _random_problem(M, N, K, g)
        buf = torch.empty(M * K + 1, dtype=torch.uint8, device=DEV)
        buf[1:] = xq.view(torch.uint8).reshape(-1).to(DEV)
        xq_off = buf[1:].view(F8).view(M, K)   # contiguous but only 1-byte aligned
        wbuf = torch.empty(N * K + 3, dtype=torch.uint8, device=DEV)
        wbuf[3:] = wq.view(torch.uint8).reshape(-1).to(DEV)
        wq_off = wbuf[3:].view(F8).view(N, K)
        ref = O.dequant_matmul(xq, wq, xs, ws)
        xs_d, ws_d = _gpu(xs, ws)
        assert_gemm_close(torch.ops.mslk.f8f8bf16_rowwise(xq_off, wq.to(DEV), xs_d, ws_d), ref)      # via the workspace copy
        assert_gemm_close(torch.ops.mslk.f8f8bf16_rowwise(xq.to(DEV), wq_off, xs_d, ws_d), ref)
        assert_gemm_close(torch.ops.mslk.f8f8f16_rowwise(xq_off, wq_off, xs_d, ws_d), ref)
        y = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)                                        # no workspace: scalar kernel
        _lib.check(_lib.lib().mslk_amd_f8f8bf16_rowwise(xq_off.data_ptr(), wq_off.data_ptr(), xs_d.data_ptr(), ws_d.data_ptr(),
                                                        None, 0, y.data_ptr(), M, N, K, None, 0, None))
        torch.cuda.synchronize()
        assert_gemm_close(y, ref)


@pytest.mark.parametrize("M,N,K", [(300, 520, 1000), (1, 8192, 8200), (16, 8192, 8190), (64, 600, 17), (5, 7, 1), (512, 4096, 1001),
                                   (1030, 2050, 4100), (40, 5200, 2047), (700, 300, 15)])
def test_k_not_a_multiple_of_16_runs_on_padded_copies(M, N, K):
    """K % 16 != 0: the ops hand the library a workspace, it copies both operands into rows of K rounded up to 16
    (zero tail) and runs the MFMA kernels on the copies.  Same tolerance as every other shape, with bias, both output
    types; through the C ABI the result without a workspace (scalar kernel) has to agree as well, and the reported
    workspace size is the documented one."""
    from mslk_amd import _lib
    g = torch.Generator().manual_seed(M + 3 * N + 5 * K)
    xq, wq, xs, ws = _random_problem(M, N, K, g)
    bias = (torch.randn(N, generator=g) * 0.5).float()
    d = _gpu(xq, wq, xs, ws)
    y = torch.ops.mslk.f8f8bf16_rowwise(*d, bias=bias.to(DEV))
    y16 = torch.ops.mslk.f8f8f16_rowwise(*d)
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    torch.ops.mslk.f8f8bf16_rowwise_out(*d, out)
    torch.cuda.synchronize()
    ref = O.dequant_matmul(xq, wq, xs, ws)
    assert_gemm_close(y, ref + bias, f"{M}x{N}x{K}")
    assert_gemm_close(y16, ref, f"fp16 {M}x{N}x{K}")
    assert_gemm_close(out, ref, f"out {M}x{N}x{K}")
    L = _lib.lib()
    Kp = (K + 15) // 16 * 16
    assert L.mslk_amd_f8f8bf16_rowwise_workspace_bytes(M, N, K) == (M + N) * Kp
    assert L.mslk_amd_f8f8bf16_rowwise_workspace_bytes(M, N, Kp) == 0
    if M * N * K <= 2 ** 31:   # the scalar kernel is slow
        y_plain = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
        _lib.check(L.mslk_amd_f8f8bf16_rowwise(d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(), None, 0,
                                               y_plain.data_ptr(), M, N, K, None, 0, None))
        small = torch.empty(16, dtype=torch.uint8, device=DEV)   # a workspace that is too small is ignored
        y_small = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
        _lib.check(L.mslk_amd_f8f8bf16_rowwise(d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(), None, 0,
                                               y_small.data_ptr(), M, N, K, small.data_ptr(), 16, None))
        torch.cuda.synchronize()
        assert_gemm_close(y_plain, ref, f"no workspace {M}x{N}x{K}")
        assert torch.equal(y_plain.view(torch.int16), y_small.view(torch.int16))


@pytest.mark.parametrize("M,N,K", [(512, 1024, 512), (16, 1024, 1024), (4352, 4352, 128), (16, 8192, 256), (64, 8192, 256),
                                   (128, 1024, 8192)])   # the last one is split along K: two launches and a workspace from the graph's pool
def test_hip_graph_capture_and_replay(M, N, K):
    """The reference tests capture + replay (test/gemm/gemm_test.py:440-447); replay several times with
    eager work in between and compare every replay with the eager result."""
    g = torch.Generator().manual_seed(24)
    xq, wq, xs, ws = _gpu(*_random_problem(M, N, K, g))
    x_bf16 = torch.randn(M, K, device=DEV).bfloat16()
    eager_q, eager_s = mslk_amd.quantize_fp8_row(x_bf16, use_triton=False)
    eager = torch.ops.mslk.f8f8bf16_rowwise(eager_q, wq, eager_s, ws)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            q, s = mslk_amd.quantize_fp8_row(x_bf16, use_triton=False)
            torch.ops.mslk.f8f8bf16_rowwise(q, wq, s, ws)
    torch.cuda.current_stream().wait_stream(side)
    with torch.cuda.graph(graph):
        q, s = mslk_amd.quantize_fp8_row(x_bf16, use_triton=False)
        y = torch.ops.mslk.f8f8bf16_rowwise(q, wq, s, ws)
    for _ in range(3):
        y.fill_(0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager)
        _ = torch.ops.mslk.f8f8bf16_rowwise(xq, wq, xs, ws)  # eager work between replays
        torch.cuda.synchronize()


def _check_sampled(y, xq, wq, xs, ws, bias, g, rows=48, what=""):
    """Full-size outputs are checked against the oracle on a seeded sample of rows."""
    M = xq.shape[0]
    idx = torch.randperm(M, generator=g)[: min(rows, M)].sort().values
    ref = O.dequant_matmul(xq[idx].cpu(), wq.cpu(), xs[idx].cpu(), ws.cpu(), None if bias is None else bias.float().cpu())
    return assert_gemm_close(y[idx.to(y.device)], ref, what)


def _quantize_gpu_checked(t_cpu, g, rows=32):
    """Quantize on the GPU and confirm a sample of rows bit-exact against the oracle."""
    q, s = mslk_amd.quantize_fp8_row(t_cpu.to(DEV), use_triton=False)
    idx = torch.randperm(t_cpu.shape[0], generator=g)[: min(rows, t_cpu.shape[0])]
    rq, rs = O.quantize_fp8_row(t_cpu[idx])
    assert torch.equal(q[idx.to(DEV)].cpu().view(torch.uint8), rq.view(torch.uint8))
    assert torch.equal(s[idx.to(DEV)].cpu().view(torch.int32), rs.view(torch.int32))
    return q, s


def test_cfg0_full():
    wl = W.cfg0()
    xq, xs = _quant_cpu(wl.x)
    wq, ws = _quant_cpu(wl.w)
    gq, gs = mslk_amd.quantize_fp8_row(wl.x.to(DEV), use_triton=False)
    assert torch.equal(gq.cpu().view(torch.uint8), xq.view(torch.uint8)) and torch.equal(gs.cpu().view(torch.int32), xs.view(torch.int32))
    y = _op(xq, wq, xs, ws)
    assert_gemm_close(y, O.dequant_matmul(xq, wq, xs, ws), "cfg0")
    # and the reference's CPU emulation path (bf16 matmul then scale) agrees within its own rounding
    cpu = O.matmul_fp8_row_cpu(xq, wq, xs, ws)
    max_rel, normwise = O.gemm_errors(y.float(), cpu.float())
    assert max_rel < 2e-2 and normwise < 8e-3


def test_cfg1_full():
    g = torch.Generator().manual_seed(101)
    wl = W.cfg1()
    xq, xs = _quantize_gpu_checked(wl.x, g, rows=4096)
    wq, ws = _quantize_gpu_checked(wl.w, g, rows=4096)
    y = torch.ops.mslk.f8f8bf16_rowwise(xq, wq, xs, ws)
    torch.cuda.synchronize()
    ref = O.dequant_matmul(xq.cpu(), wq.cpu(), xs.cpu(), ws.cpu())
    assert_gemm_close(y, ref, "cfg1")


def test_cfg2_full_with_bias():
    g = torch.Generator().manual_seed(102)
    wl = W.cfg2()
    xq, xs = _quantize_gpu_checked(wl.x, g)
    wq, ws = _quantize_gpu_checked(wl.w, g)
    bias = wl.bias.to(DEV)
    y = torch.ops.mslk.f8f8bf16_rowwise(xq, wq, xs, ws, bias=bias)
    torch.cuda.synchronize()
    assert y.shape == (8192, 28672)
    # the WHOLE output against the fp32 oracle, in blocks of 1024 rows (1.9 TFLOP of CPU work in all): every tile, every
    # tile edge and every pass of the persistent workgroups is covered, not a sample of rows
    wq_c, ws_c, bias_c = wq.cpu(), ws.cpu(), bias.float().cpu()
    wd = wq_c.float() * ws_c[:, None]                      # dequantized once
    for r0 in range(0, 8192, 1024):
        rows = slice(r0, r0 + 1024)
        ref = (xq[rows].cpu().float() * xs[rows].cpu()[:, None]) @ wd.t() + bias_c[None, :]
        assert_gemm_close(y[rows], ref, f"cfg2 rows {r0}..{r0 + 1023}")
    del wd
    # linearity in the scales (size-independent property): doubling x_scale doubles y - bias exactly in fp32,
    # so the two bf16 outputs differ by at most one rounding
    y2 = torch.ops.mslk.f8f8bf16_rowwise(xq, wq, xs * 2, ws, bias=bias)
    sl = slice(0, 256)
    a = (y2[sl].float() - bias.float()[None, :]) / 2
    b = y[sl].float() - bias.float()[None, :]
    assert torch.allclose(a, b, rtol=1.6e-2, atol=1e-2)


@pytest.mark.parametrize("M", [1, 4, 16, 64])
def test_cfg3_decode(M):
    g = torch.Generator().manual_seed(103)
    w = W.cfg3_weight()
    wq, ws = _quantize_gpu_checked(w, g)
    x = W.cfg3_activations(M)
    xq, xs = mslk_amd.quantize_fp8_row(x.to(DEV), use_triton=False)
    rq, rs = O.quantize_fp8_row(x)
    assert torch.equal(xq.cpu().view(torch.uint8), rq.view(torch.uint8)) and torch.equal(xs.cpu().view(torch.int32), rs.view(torch.int32))
    y = torch.ops.mslk.f8f8bf16_rowwise(xq, wq, xs, ws)
    torch.cuda.synchronize()
    ref = O.dequant_matmul(rq, wq.cpu(), rs, ws.cpu())
    assert_gemm_close(y, ref, f"cfg3 M={M}")
    # the same step as ONE operator (one launch for M <= 4): quantized on the fly, same codes and scales, same tolerance
    y1, xq1, xs1 = torch.ops.mslk.quantize_f8f8bf16_rowwise(x.to(DEV), wq, ws)
    torch.cuda.synchronize()
    assert torch.equal(xq1.cpu().view(torch.uint8), rq.view(torch.uint8)) and torch.equal(xs1.cpu().view(torch.int32), rs.view(torch.int32))
    assert_gemm_close(y1, ref, f"cfg3 M={M}, quantizer fused")


@pytest.mark.parametrize("M,N,K", [(512, 512, 256), (300, 260, 384), (16, 512, 512), (40, 300, 1040), (33, 20, 50),
                                   (1, 8192, 1024), (2048, 1024, 512)])
def test_fp16_output_exact_cases_and_overflow(M, N, K):
    """f8f8f16_rowwise on inputs whose fp32 result is exact: the output must be the fp16 rounding
    (nearest even, overflow to infinity) of that result, bit for bit.  The scales reach 2^6, so some
    outputs exceed 65504 and must come out infinite."""
    g = torch.Generator().manual_seed(K + 1)
    xi = torch.randint(-8, 9, (M, K), generator=g).float()
    wi = torch.randint(-8, 9, (N, K), generator=g).float()
    xs = 2.0 ** torch.randint(-9, 7, (M,), generator=g).float()
    ws = 2.0 ** torch.randint(-9, 7, (N,), generator=g).float()
    bias = torch.randint(-4, 5, (N,), generator=g).float() * 2.0 ** -5
    want = ((xi @ wi.T) * xs[:, None] * ws[None, :] + bias[None, :]).to(torch.float16)
    y = torch.ops.mslk.f8f8f16_rowwise(*_gpu(xi.to(F8), wi.to(F8), xs, ws), bias=bias.to(DEV))
    torch.cuda.synchronize()
    assert y.dtype == torch.float16 and y.shape == (M, N)
    assert torch.equal(y.cpu().view(torch.int16), want.view(torch.int16))
    if M * N >= 512 * 512:
        assert torch.isinf(want).any() and (want.abs() < 2.0 ** -14).any()   # overflow and subnormal results both occur


@pytest.mark.parametrize("M,N,K", [(4096, 4096, 4096), (300, 517, 256), (64, 8192, 8192), (5, 8200, 5120), (65, 33, 17)])
def test_fp16_output_matches_oracle(M, N, K):
    g = torch.Generator().manual_seed(M + N + K)
    xq, wq, xs, ws = _random_problem(M, N, K, g)
    y = torch.ops.mslk.f8f8f16_rowwise(*_gpu(xq, wq, xs, ws))
    yb = torch.ops.mslk.f8f8bf16_rowwise(*_gpu(xq, wq, xs, ws))
    torch.cuda.synchronize()
    ref = O.dequant_matmul(xq, wq, xs, ws)
    assert_gemm_close(y, ref, "fp16 out")
    _, normwise = O.gemm_errors(y.float().cpu(), ref)
    assert normwise <= 5e-4   # fp16 keeps 10 mantissa bits: only the accumulation error is left
    # both outputs are roundings of the same fp32 value v: |fp16(v) - v| <= 2^-11 |v| and |bf16(v) - v| <= 2^-8 |v|,
    # and re-rounding the fp16 result to bf16 lands on another bf16 than the direct rounding only when
    # v lies within half an fp16 ulp of a bf16 rounding boundary (1 value in 16 for a smooth distribution)
    yf, ybf = y.float(), yb.float()
    normal = yf.abs() >= 2.0 ** -14
    assert ((yf - ybf).abs()[normal] <= yf.abs()[normal] * (2.0 ** -8 + 2.0 ** -11) * 1.0001).all()
    differs = (yf.bfloat16() != yb).float().mean().item()
    assert differs < 0.09


def test_seeded_random_shape_sweep():
    """Sixty seeded shapes across the dispatch boundaries (skinny <-> tiled at M = 64, 128^2 <-> 256^2 tiles,
    K tails, K % 16 != 0 -> generic kernel, N not a multiple of 8), with and without bias, both output types."""
    g = torch.Generator().manual_seed(2024)
    for case in range(60):
        M = int(torch.randint(1, 400, (1,), generator=g))
        N = int(torch.randint(1, 700, (1,), generator=g))
        K = int(torch.randint(1, 80, (1,), generator=g)) * (16 if case % 5 else 1)
        if case % 7 == 0:
            M, N = M * 9, N * 5          # enough tiles for the 256 x 256 shape
        xq, wq, xs, ws = _random_problem(M, N, K, g)
        bias = (torch.randn(N, generator=g) * 0.5).to(torch.bfloat16 if case % 2 else torch.float32) if case % 3 == 0 else None
        op = torch.ops.mslk.f8f8f16_rowwise if case % 4 == 1 else torch.ops.mslk.f8f8bf16_rowwise
        y = op(*_gpu(xq, wq, xs, ws), bias=None if bias is None else bias.to(DEV))
        torch.cuda.synchronize()
        ref = O.dequant_matmul(xq, wq, xs, ws, None if bias is None else bias.float())
        assert y.shape == (M, N)
        assert_gemm_close(y, ref, f"case {case}: {M}x{N}x{K} bias={None if bias is None else bias.dtype} op={op}")


@pytest.mark.parametrize("M,N,K", [(65, 8192, 8192), (128, 4096, 4096), (200, 2048, 4096), (256, 1024, 8192), (100, 520, 2064),
                                   (384, 4096, 2048), (128, 1024, 14336), (96, 16384, 2048), (130, 64, 272), (70, 136, 144),
                                   (512, 8192, 1024), (66, 72, 16), (65, 4096, 1024), (96, 8192, 400), (128, 7176, 272),
                                   (250, 4096, 144), (129, 4104, 2048), (100, 6144, 128), (1000, 8192, 272), (1536, 4104, 144),
                                   (2048, 5120, 128), (1536, 6144, 144), (1500, 6152, 128), (128, 57344, 128), (100, 50000, 144),
                                   (384, 20480, 128)])
def test_medium_m_shapes_use_narrow_and_ring_tiles(M, N, K):
    """Shapes between the skinny kernel (M <= 64) and a full grid of 256 x 256 tiles: 128 x 32 / 128 x 64 / 128 x 128
    tiles with deep operand rings.  Oracle tolerance, both output types, bias, and the pre-shuffled weights."""
    g = torch.Generator().manual_seed(M * 3 + N + K)
    xq, wq, xs, ws = _random_problem(M, N, K, g)
    bias = (torch.randn(N, generator=g) * 0.5).float()
    d = _gpu(xq, wq, xs, ws)
    y = torch.ops.mslk.f8f8bf16_rowwise(*d, bias=bias.to(DEV))
    y16 = torch.ops.mslk.f8f8f16_rowwise(*d)
    torch.cuda.synchronize()
    assert_gemm_close(y, O.dequant_matmul(xq, wq, xs, ws, bias), f"{M}x{N}x{K}")
    assert_gemm_close(y16, O.dequant_matmul(xq, wq, xs, ws), f"fp16 {M}x{N}x{K}")
    if N % 16 == 0 and K % 64 == 0:
        yp = torch.ops.mslk.f8f8bf16_rowwise_preshuffle(d[0], mslk_amd.preshuffle_b_mfma(d[1]), d[2], d[3], bias=bias.to(DEV))
        torch.cuda.synchronize()
        assert_gemm_close(yp, O.dequant_matmul(xq, wq, xs, ws, bias), f"pre-shuffled {M}x{N}x{K}")


@pytest.mark.parametrize("M,N,K", [(4352, 4352, 256), (4100, 4500, 400), (8192, 2304, 128), (2304, 8200, 48), (5000, 4608, 144),
                                   (2304, 8192, 128), (4609, 4096, 144), (650, 28672, 64), (2561, 8200, 272)])
def test_more_tiles_than_compute_units(M, N, K):
    """More than 256 tiles of 256 x 256: one persistent workgroup per CU walks several tiles, fetching the next
    tile's first operands before the epilogue of the current one.  Ragged last rows / columns, K tails, one-step and
    zero-step K loops, both bias types, both output types and the pre-shuffled weights against the oracle.  The last
    four shapes leave a last pass less than half full, whose rows a second launch computes with smaller tiles."""
    assert ((M + 255) // 256) * ((N + 255) // 256) > 256
    g = torch.Generator().manual_seed(M + 7 * N + K)
    xq, wq, xs, ws = _random_problem(M, N, K, g)
    bias = (torch.randn(N, generator=g) * 0.5).float()
    d = _gpu(xq, wq, xs, ws)
    y = torch.ops.mslk.f8f8bf16_rowwise(*d, bias=bias.to(DEV))
    yb = torch.ops.mslk.f8f8bf16_rowwise(*d, bias=bias.bfloat16().to(DEV))
    y16 = torch.ops.mslk.f8f8f16_rowwise(*d)
    torch.cuda.synchronize()
    ref = O.dequant_matmul(xq, wq, xs, ws)
    assert_gemm_close(y, ref + bias, f"{M}x{N}x{K}")
    assert_gemm_close(yb, ref + bias.bfloat16().float(), f"bf16 bias {M}x{N}x{K}")
    assert_gemm_close(y16, ref, f"fp16 {M}x{N}x{K}")
    if N % 16 == 0 and K % 64 == 0:
        yp = torch.ops.mslk.f8f8bf16_rowwise_preshuffle(d[0], mslk_amd.preshuffle_b_mfma(d[1]), d[2], d[3])
        torch.cuda.synchronize()
        assert_gemm_close(yp, ref, f"pre-shuffled {M}x{N}x{K}")


@pytest.mark.parametrize("M,N,K", [(9, 8192, 1024), (16, 8200, 512), (32, 16384, 384), (24, 20000, 272), (33, 8192, 2048),
                                   (48, 12296, 144), (64, 9000, 1040), (64, 16383, 128), (40, 28672, 256), (17, 8192, 16),
                                   (12, 5120, 1024), (64, 6152, 400), (31, 7168, 2048), (48, 9216, 272), (64, 20488, 144),
                                   (33, 57344, 128), (64, 8200, 1024)])
def test_small_m_on_wide_weights_uses_short_tiles(M, N, K):
    """8 < M <= 64 with N >= 5120 and row-major weights: 32 x 32, 64 x 32 and (32 < M, N > 8192) 64 x 64 tiles (two- and
    four-wave workgroups, deep operand rings) instead of the weight-streaming kernel.  Ragged rows and columns, K tails, bias, fp16 output."""
    g = torch.Generator().manual_seed(M * 5 + N + K)
    xq, wq, xs, ws = _random_problem(M, N, K, g)
    bias = (torch.randn(N, generator=g) * 0.5).float()
    d = _gpu(xq, wq, xs, ws)
    y = torch.ops.mslk.f8f8bf16_rowwise(*d, bias=bias.to(DEV))
    y16 = torch.ops.mslk.f8f8f16_rowwise(*d)
    torch.cuda.synchronize()
    ref = O.dequant_matmul(xq, wq, xs, ws)
    assert_gemm_close(y, ref + bias, f"{M}x{N}x{K}")
    assert_gemm_close(y16, ref, f"fp16 {M}x{N}x{K}")


def test_seeded_random_sweep_small_m_wide_n():
    """Forty seeded shapes with M <= 96 and N around and above the width from which short tiles replace the
    weight-streaming kernel (M = 8 / 9, 32 / 33, 64 / 65; N = 4096 ... 20000; K with and without tails), row-major and
    pre-shuffled weights, with and without bias, both output types."""
    g = torch.Generator().manual_seed(77)
    edges_m = [1, 8, 9, 16, 31, 32, 33, 48, 63, 64, 65, 96]
    for case in range(40):
        M = edges_m[case % len(edges_m)] if case % 3 else int(torch.randint(1, 97, (1,), generator=g))
        N = int(torch.randint(4096 // 8, 20000 // 8, (1,), generator=g)) * 8
        if case % 4 == 0:
            N = N // 16 * 16
        K = int(torch.randint(1, 24, (1,), generator=g)) * (64 if case % 2 else 16)
        xq, wq, xs, ws = _random_problem(M, N, K, g)
        bias = (torch.randn(N, generator=g) * 0.5).to(torch.bfloat16 if case % 2 else torch.float32) if case % 3 == 0 else None
        d = _gpu(xq, wq, xs, ws)
        ref = O.dequant_matmul(xq, wq, xs, ws, None if bias is None else bias.float())
        op = torch.ops.mslk.f8f8f16_rowwise if case % 5 == 1 else torch.ops.mslk.f8f8bf16_rowwise
        y = op(*d, bias=None if bias is None else bias.to(DEV))
        torch.cuda.synchronize()
        assert_gemm_close(y, ref, f"case {case}: {M}x{N}x{K} op={op}")
        if N % 16 == 0 and K % 64 == 0:
            yp = torch.ops.mslk.f8f8bf16_rowwise_preshuffle(d[0], mslk_amd.preshuffle_b_mfma(d[1]), d[2], d[3],
                                                            bias=None if bias is None else bias.to(DEV))
            torch.cuda.synchronize()
            assert_gemm_close(yp, ref, f"case {case} pre-shuffled: {M}x{N}x{K}")


@pytest.mark.parametrize("M,N,K", [(64, 512, 1024), (300, 520, 640), (1024, 1024, 512)])
def test_matches_the_model_level_fake_quant_statement(M, N, K):
    """The reference states the same semantics a second time in its MoE baseline (mslk/moe/layers.py:476-488):
    y = bf16( bf16_matmul(xq.bf16, wq.bf16^T) * xs[:, None] * ws[None, :] ).  e4m3 values are exact in bf16, so that
    expression differs from the kernel's only by the bf16 rounding of the un-scaled matmul: one more rounding of
    2^-9 relative."""
    g = torch.Generator().manual_seed(M + N + K)
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) * 0.05).bfloat16()
    xq, xs = O.quantize_fp8_row(x)
    wq, ws = O.quantize_fp8_row(w)
    y = torch.ops.mslk.f8f8bf16_rowwise(*_gpu(xq, wq, xs, ws))
    torch.cuda.synchronize()
    stated = (torch.matmul(xq.to(torch.bfloat16), wq.to(torch.bfloat16).t()) * xs[:, None] * ws[None, :]).to(torch.bfloat16)
    err = (y.float().cpu() - stated.float()).abs()
    # two bf16 roundings apart at most; results that cancel to almost nothing also see the accumulation order
    assert (err <= stated.float().abs() * 2.0 ** -7 + stated.float().abs().max() * 2.0 ** -10).all()
    max_rel, normwise = O.gemm_errors(y.float().cpu(), stated.float())
    assert max_rel <= O.MAX_REL_TOL and normwise <= 2 * O.NORMWISE_TOL


@pytest.mark.parametrize("M,N,K,bias_dtype", [(1, 512, 1024, None), (3, 1000, 2048, torch.bfloat16), (4, 8200, 5120, torch.float32),
                                              (2, 48, 3072, None), (4, 16, 8192, torch.bfloat16), (2, 4096, 14336, None),
                                              (1, 520, 15360, None), (3, 300, 16384, None),
                                              (2, 4096, 11008, None), (4, 1000, 13824, torch.bfloat16), (1, 264, 1152, None),   # K steps that do not divide among the waves
                                              (7, 520, 2048, None), (4, 300, 1040, torch.bfloat16)])   # the last two: two launches
def test_quantize_fused_into_the_decode_gemm(M, N, K, bias_dtype):
    """quantize_f8f8bf16_rowwise: codes and scales are the stand-alone quantizer's bits (checked against the oracle),
    the product meets the GEMM tolerance; rows of zeros, a NaN and an infinity behave as in the quantizer; the
    activations may be a strided view."""
    g = torch.Generator().manual_seed(M * 1000003 + N * 101 + K)
    base = torch.randn(M, K + 24, generator=g).bfloat16()
    x = base[:, 8:8 + K]                                   # row stride K + 24 elements, 16-byte aligned rows
    if M >= 3:
        x[1].zero_()
    if M >= 4:
        x[2, 17] = float("nan")
        x[3, 100] = float("inf")
    w = (torch.randn(N, K, generator=g) * 0.02).bfloat16()
    wq, ws = O.quantize_fp8_row(w)
    bias = None if bias_dtype is None else (torch.randn(N, generator=g) * 0.05).to(bias_dtype)
    xd = base.to(DEV)[:, 8:8 + K]
    y, xq, xs = torch.ops.mslk.quantize_f8f8bf16_rowwise(xd, wq.to(DEV), ws.to(DEV), None if bias is None else bias.to(DEV))
    torch.cuda.synchronize()
    assert y.shape == (M, N) and y.dtype == torch.bfloat16 and xq.shape == (M, K) and xs.shape == (M,)
    assert_quant_bit_exact(x.contiguous(), xq, xs)
    rq, rs = O.quantize_fp8_row(x.contiguous())
    finite = torch.isfinite(rs) & ~torch.isnan(rq.float()).any(dim=1)
    ref = O.dequant_matmul(rq[finite], wq, rs[finite], ws, None if bias is None else bias.float())
    assert_gemm_close(y[finite.to(DEV)], ref, f"fused {M}x{N}x{K}")
    if (~finite).any():
        assert torch.isnan(y[(~finite).to(DEV)].float()).any(dim=1).all()


def test_quantize_fused_gives_the_quantizer_bits_for_negative_nan_and_infinity():
    """The codes and scales the one-launch path writes out are the stand-alone quantizer's for every input: rows with
    -NaN, -inf, +NaN and +inf elements are compared byte for byte (sign bits of the NaN codes included) with
    quantize_fp8_row(use_triton=False) on the same device."""
    g = torch.Generator().manual_seed(5)
    M, N, K = 4, 520, 2048
    x = torch.randn(M, K, generator=g).bfloat16()
    bits = x.view(torch.int16)
    bits[0, 33] = -64            # 0xFFC0: negative quiet NaN
    bits[1, 1000] = -128         # 0xFF80: -inf
    bits[2, 5] = 0x7FC0          # +NaN ...
    bits[2, 6] = -128            # ... and -inf in the same row
    x[3, 77] = float("inf")
    x[3, 78] = -3.0
    wq, ws = O.quantize_fp8_row((torch.randn(N, K, generator=g) * 0.02).bfloat16())
    xd = x.to(DEV)
    y, xq, xs = torch.ops.mslk.quantize_f8f8bf16_rowwise(xd, wq.to(DEV), ws.to(DEV))
    q2, s2 = mslk_amd.quantize_fp8_row(xd, use_triton=False)
    torch.cuda.synchronize()
    assert torch.equal(xq.view(torch.uint8), q2.view(torch.uint8)), "codes differ from the stand-alone quantizer"
    assert torch.equal(xs.view(torch.int32), s2.view(torch.int32)), "scale bits differ from the stand-alone quantizer"
    assert (xq.view(torch.uint8)[0] & 0x7F == 0x7F).all() and torch.isnan(xs[0])   # a NaN row is NaN codes throughout


def test_quantize_fused_graph_capture():
    g = torch.Generator().manual_seed(77)
    x = torch.randn(4, 4096, generator=g).bfloat16().to(DEV)
    wq, ws = mslk_amd.quantize_fp8_row((torch.randn(1024, 4096, generator=g) * 0.02).bfloat16().to(DEV), use_triton=False)
    eager = torch.ops.mslk.quantize_f8f8bf16_rowwise(x, wq, ws)[0].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        torch.ops.mslk.quantize_f8f8bf16_rowwise(x, wq, ws)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y, q, s = torch.ops.mslk.quantize_f8f8bf16_rowwise(x, wq, ws)
    for _ in range(3):
        y.fill_(7.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager)


@pytest.mark.parametrize("N,K", [(8, 1 << 25), (4, 1 << 26)])
def test_rows_longer_than_the_streaming_kernels_32_bit_offsets(N, K):
    """The weight-streaming kernel forms 32-bit byte offsets of up to 63 * K + k: K = 2^25 is the last power of two it
    may take, K = 2^26 has to go to a kernel with 64-bit addressing.  Either way every weight row must be read where it
    lies (rows differ, so a wrapped offset would show)."""
    g = torch.Generator(device=DEV).manual_seed(N + (K >> 20))
    def codes(*shape):
        mag = torch.randint(0x20, 0x48, shape, dtype=torch.uint8, device=DEV, generator=g)     # |value| in [0.125, 4)
        sign = torch.randint(0, 2, shape, dtype=torch.uint8, device=DEV, generator=g) << 7
        return (mag | sign).view(F8)
    xq, wq = codes(1, K), codes(N, K)
    xs = torch.full((1,), 2.0 ** -8, device=DEV)
    ws = torch.rand(N, device=DEV, generator=g) * 1e-3 + 1e-3
    y = torch.ops.mslk.f8f8bf16_rowwise(xq, wq, xs, ws)
    torch.cuda.synchronize()
    ref = torch.zeros(N, dtype=torch.float64, device=DEV)
    step = 1 << 22
    for k0 in range(0, K, step):
        ref += (wq[:, k0:k0 + step].float() * xq[:, k0:k0 + step].float()).double().sum(dim=1)
    ref = (ref * ws.double() * xs.double()).float().view(1, N)
    assert_gemm_close(y.cpu(), ref.cpu(), f"N={N} K={K}")
