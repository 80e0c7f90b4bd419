"""GPU parity of the offsets-based grouped GEMM (all four operand-rank combinations) and of the
batched GEMM: every group must match the oracle's dense dequantised product of the slices the
group owns, which is how test/gemm/gemm_test.py:519-600 (batched, 3D-3D) and 603-856 (3D-2D,
2D-2D, 2D-3D) validate the reference (a loop of per-group matmuls)."""
import pytest
import torch

import mslk_amd  # noqa: F401  (registers torch.ops.mslk.*)
from oracle import fp8_rowwise_oracle as O
from tests.helpers import assert_gemm_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F8 = torch.float8_e4m3fn
SENTINEL = -7.0


def _quant(rows, K, g, scale=1.0):
    if rows == 0:
        return torch.empty(0, K, dtype=F8), torch.empty(0)
    return O.quantize_fp8_row((torch.randn(rows, K, generator=g) * scale).bfloat16())


def _ends(sizes):
    return torch.tensor(sizes, dtype=torch.int64).cumsum(0).to(torch.int32).to(DEV)


def _sentinel(*shape):
    return torch.full(shape, SENTINEL, dtype=torch.bfloat16, device=DEV)


@pytest.mark.parametrize("ms,N,K,extra", [
    ([64], 512, 512, 0), ([300, 0, 17, 256, 1], 768, 512, 0), ([0, 0, 5], 512, 1024, 3),
    ([128] * 16, 1024, 512, 0), ([7, 300, 0, 0, 513, 64, 2, 1000], 520, 656, 40), ([1] * 16, 264, 144, 0),
    ([700, 900], 2048, 512, 0),   # large enough average group for 256 x 256 tiles
])
def test_2d_3d_offsets_over_m(ms, N, K, extra):
    g = torch.Generator().manual_seed(sum(ms) + N + K)
    total = sum(ms) + extra   # `extra` rows lie beyond the last offset and must stay untouched
    xq, xs = _quant(total, K, g)
    wq, ws = _quant(len(ms) * N, K, g, 0.02)
    out = _sentinel(total, N)
    y = torch.ops.mslk.f8f8bf16_rowwise_grouped_mm(xq.to(DEV), wq.view(len(ms), N, K).to(DEV), xs.to(DEV),
                                                   ws.view(len(ms), N).to(DEV), _ends(ms), out)
    torch.cuda.synchronize()
    assert y.data_ptr() == out.data_ptr()
    r0 = 0
    for gi, m in enumerate(ms):
        if m:
            ref = O.dequant_matmul(xq[r0:r0 + m], wq[gi * N:(gi + 1) * N], xs[r0:r0 + m], ws[gi * N:(gi + 1) * N])
            assert_gemm_close(y[r0:r0 + m], ref, f"group {gi}")
        r0 += m
    assert (y[r0:] == SENTINEL).all()
    # the int64-sizes entry point on the same data gives the same bits
    if extra == 0 and N >= 512 and K >= 512:
        y2 = torch.ops.mslk.f8f8bf16_rowwise_grouped_stacked(xq.to(DEV), wq.view(len(ms), N, K).to(DEV), xs.to(DEV),
                                                             ws.view(len(ms), N).to(DEV),
                                                             torch.tensor(ms, dtype=torch.int64, device=DEV))
        torch.cuda.synchronize()
        assert torch.equal(y2, y)


@pytest.mark.parametrize("ns,M,K,extra", [
    ([64], 512, 512, 0), ([64, 128, 8, 0, 200], 300, 512, 0), ([512] * 4, 100, 272, 16),
    ([5, 3, 17, 40], 70, 256, 0),   # column blocks that start at unaligned addresses of the output
    ([1024, 768], 1500, 512, 0),
])
def test_3d_2d_offsets_over_n(ns, M, K, extra):
    g = torch.Generator().manual_seed(sum(ns) + M + K)
    G, total = len(ns), sum(ns) + extra
    xq, xs = _quant(G * M, K, g)
    wq, ws = _quant(total, K, g, 0.02)
    out = _sentinel(M, total)
    y = torch.ops.mslk.f8f8bf16_rowwise_grouped_mm(xq.view(G, M, K).to(DEV), wq.to(DEV), xs.view(G, M).to(DEV),
                                                   ws.to(DEV), _ends(ns), out)
    torch.cuda.synchronize()
    c0 = 0
    for gi, n in enumerate(ns):
        if n:
            ref = O.dequant_matmul(xq[gi * M:(gi + 1) * M], wq[c0:c0 + n], xs[gi * M:(gi + 1) * M], ws[c0:c0 + n])
            assert_gemm_close(y[:, c0:c0 + n], ref, f"group {gi}")
        c0 += n
    assert (y[:, c0:] == SENTINEL).all()


@pytest.mark.parametrize("G,M,N,K", [(1, 512, 512, 512), (4, 100, 520, 272), (16, 64, 512, 512), (3, 3, 8, 16),
                                     (5, 300, 1032, 1024), (8, 1024, 1024, 512)])
def test_3d_3d_and_batched(G, M, N, K):
    g = torch.Generator().manual_seed(G + M + N + K)
    xq, xs = _quant(G * M, K, g)
    wq, ws = _quant(G * N, K, g, 0.02)
    XQ, WQ = xq.view(G, M, K).to(DEV), wq.view(G, N, K).to(DEV)
    XS, WS = xs.view(G, M).to(DEV), ws.view(G, N).to(DEV)
    out = _sentinel(G, M, N)
    y = torch.ops.mslk.f8f8bf16_rowwise_grouped_mm(XQ, WQ, XS, WS, None, out)
    yb = torch.ops.mslk.f8f8bf16_rowwise_batched(XQ, WQ, XS, WS)
    bias32 = torch.randn(G, N, generator=g)
    yb32 = torch.ops.mslk.f8f8bf16_rowwise_batched(XQ, WQ, XS, WS, bias32.to(DEV))
    out2 = _sentinel(G, M, N)
    yb16 = torch.ops.mslk.f8f8bf16_rowwise_batched(XQ, WQ, XS, WS, bias32.bfloat16().to(DEV), True, out2)
    torch.cuda.synchronize()
    assert yb16.data_ptr() == out2.data_ptr() and yb.shape == (G, M, N) and yb.dtype == torch.bfloat16
    assert torch.equal(y, yb)
    for gi in range(G):
        sl_m, sl_n = slice(gi * M, (gi + 1) * M), slice(gi * N, (gi + 1) * N)
        assert_gemm_close(y[gi], O.dequant_matmul(xq[sl_m], wq[sl_n], xs[sl_m], ws[sl_n]), f"batch {gi}")
        assert_gemm_close(yb32[gi], O.dequant_matmul(xq[sl_m], wq[sl_n], xs[sl_m], ws[sl_n], bias32[gi]), f"batch {gi} fp32 bias")
        assert_gemm_close(yb16[gi], O.dequant_matmul(xq[sl_m], wq[sl_n], xs[sl_m], ws[sl_n], bias32[gi].bfloat16()),
                          f"batch {gi} bf16 bias")


@pytest.mark.parametrize("ks,M,N", [
    ([512] * 4, 300, 264), ([128, 0, 256, 48], 130, 512), ([512], 512, 512),
    ([100, 28, 7, 121], 40, 72),        # slices that are not 16-byte multiples take the scalar tile path
    ([1024, 2048], 1100, 1024),
    ([100, 30], 33, 40),                # total K not a multiple of 16 either
])
def test_2d_2d_offsets_over_k(ks, M, N):
    g = torch.Generator().manual_seed(sum(ks) + M + N)
    G = len(ks)
    xqs, xss, wqs, wss = [], [], [], []
    for k in ks:   # every group is quantised on its own K slice, as gemm_test.py:676-699 does
        if k:
            q, s = _quant(M, k, g); xqs.append(q); xss.append(s)
            q, s = _quant(N, k, g, 0.02); wqs.append(q); wss.append(s)
        else:
            xqs.append(torch.empty(M, 0, dtype=F8)); xss.append(torch.ones(M))
            wqs.append(torch.empty(N, 0, dtype=F8)); wss.append(torch.ones(N))
    XQ = torch.cat([q.view(torch.uint8) for q in xqs], dim=1).view(F8).contiguous().to(DEV)
    WQ = torch.cat([q.view(torch.uint8) for q in wqs], dim=1).view(F8).contiguous().to(DEV)
    out = _sentinel(G, M, N)
    y = torch.ops.mslk.f8f8bf16_rowwise_grouped_mm(XQ, WQ, torch.cat(xss).to(DEV), torch.cat(wss).to(DEV), _ends(ks), out)
    torch.cuda.synchronize()
    for gi, k in enumerate(ks):
        if k:
            assert_gemm_close(y[gi], O.dequant_matmul(xqs[gi], wqs[gi], xss[gi], wss[gi]), f"group {gi}")
        else:
            assert (y[gi] == 0).all()   # empty sum


@pytest.mark.parametrize("G,M,N,K,live", [(4, 300, 512, 512, [300, 0, 17, 256]), (2, 64, 768, 1024, [1, 64]),
                                          (3, 700, 520, 656, [513, 700, 255])])
def test_grouped_dynamic_prepadded_rows(G, M, N, K, live):
    g = torch.Generator().manual_seed(G + M + N + K)
    xq, xs = _quant(G * M, K, g)
    wq, ws = _quant(G * N, K, g, 0.02)
    zs = torch.tensor(live, dtype=torch.int64, device=DEV)
    y = torch.ops.mslk.f8f8bf16_rowwise_grouped_dynamic(xq.view(G, M, K).to(DEV), wq.view(G, N, K).to(DEV),
                                                        xs.view(G, M).to(DEV), ws.view(G, N).to(DEV), zs)
    torch.cuda.synchronize()
    assert y.shape == (G, M, N) and y.dtype == torch.bfloat16
    for gi, m in enumerate(live):
        if m:
            rows, cols = slice(gi * M, gi * M + m), slice(gi * N, (gi + 1) * N)
            assert_gemm_close(y[gi, :m], O.dequant_matmul(xq[rows], wq[cols], xs[rows], ws[cols]), f"group {gi}")
        assert (y[gi, m:] == 0).all()


def test_inconsistent_offsets_write_nothing_out_of_range():
    g = torch.Generator().manual_seed(5)
    M, N, K = 128, 512, 512
    xq, xs = _quant(M, K, g)
    wq, ws = _quant(2 * N, K, g, 0.02)
    out = _sentinel(M, N)
    ends = torch.tensor([64, 10000], dtype=torch.int32, device=DEV)   # second group claims rows that do not exist
    torch.ops.mslk.f8f8bf16_rowwise_grouped_mm(xq.to(DEV), wq.view(2, N, K).to(DEV), xs.to(DEV), ws.view(2, N).to(DEV), ends, out)
    torch.cuda.synchronize()
    assert_gemm_close(out[:64], O.dequant_matmul(xq[:64], wq[:N], xs[:64], ws[:N]))
    assert (out[64:] == SENTINEL).all()


def test_groups_after_an_inconsistent_one_take_no_workgroups_from_the_valid_ones():
    """Offsets [M, 0, M, 0, M, 0]: group 0 owns every row, group 1 ends before it starts, and the groups after it look
    valid again.  Every tile of group 0 must be computed (the tile count that cuts the list into XCD slices stops at the
    first bad group; counting the later ones would leave tiles of group 0 without a workgroup) and nothing else touched."""
    g = torch.Generator().manual_seed(7)
    M, N, K, G = 2048, 512, 512, 6
    xq, xs = _quant(M, K, g)
    wq, ws = _quant(G * N, K, g, 0.02)
    out = _sentinel(M, N)
    ends = torch.tensor([M, 0, M, 0, M, 0], dtype=torch.int32, device=DEV)
    torch.ops.mslk.f8f8bf16_rowwise_grouped_mm(xq.to(DEV), wq.view(G, N, K).to(DEV), xs.to(DEV), ws.view(G, N).to(DEV), ends, out)
    torch.cuda.synchronize()
    assert not (out == SENTINEL).all(dim=1).any(), "rows of the valid first group were left uncomputed"
    assert_gemm_close(out, O.dequant_matmul(xq, wq[:N], xs, ws[:N]))


@pytest.mark.parametrize("sizes", [[64, 10000], [64, 2 ** 40], [64, -3, 20], [64] + [2 ** 30] * 4 + [32], [2 ** 31 - 1, 2 ** 31 - 1, 2]])
def test_inconsistent_sizes_of_the_stacked_entry_point_write_nothing_out_of_range(sizes):
    """int64 group sizes that do not fit the tensor (too large, negative, or adding up past 2^31 so that a 32-bit running sum
    would wrap): groups before the first bad one are computed, nothing else is touched."""
    from mslk_amd import _lib
    g = torch.Generator().manual_seed(6)
    M, N, K, G = 128, 512, 512, len(sizes)
    xq, xs = _quant(M, K, g)
    wq, ws = _quant(G * N, K, g, 0.02)
    out = _sentinel(M, N)
    dev = [t.to(DEV) for t in (xq, wq, xs, ws)]
    msz = torch.tensor(sizes, dtype=torch.int64, device=DEV)
    _lib.check(_lib.lib().mslk_amd_f8f8bf16_rowwise_grouped_stacked(dev[0].data_ptr(), dev[1].data_ptr(), dev[2].data_ptr(),
                                                                    dev[3].data_ptr(), msz.data_ptr(), G, M, N, K, out.data_ptr(),
                                                                    torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    good = sizes[0] if 0 <= sizes[0] <= M else 0
    if good:
        assert_gemm_close(out[:good], O.dequant_matmul(xq[:good], wq[:N], xs[:good], ws[:N]))
    assert (out[good:] == SENTINEL).all()


def test_argument_checks_follow_the_reference():
    XQ = torch.zeros(64, 512, dtype=F8, device=DEV)
    WQ = torch.zeros(2, 512, 512, dtype=F8, device=DEV)
    xs, ws = torch.ones(64, device=DEV), torch.ones(2, 512, device=DEV)
    out = torch.empty(64, 512, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="Must pass offsets"):
        torch.ops.mslk.f8f8bf16_rowwise_grouped_mm(XQ, WQ, xs, ws, None, out)
    with pytest.raises(RuntimeError, match="offsets must be int32"):
        torch.ops.mslk.f8f8bf16_rowwise_grouped_mm(XQ, WQ, xs, ws, torch.tensor([32, 64], device=DEV), out)
    with pytest.raises(RuntimeError, match="out shape must be"):
        torch.ops.mslk.f8f8bf16_rowwise_grouped_mm(XQ, WQ, xs, ws, torch.tensor([32, 64], dtype=torch.int32, device=DEV),
                                                   torch.empty(64, 256, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(RuntimeError, match="Offsets should not be passed"):
        torch.ops.mslk.f8f8bf16_rowwise_grouped_mm(XQ.view(2, 32, 512), WQ, xs.view(2, 32), ws,
                                                   torch.tensor([32, 64], dtype=torch.int32, device=DEV),
                                                   torch.empty(2, 32, 512, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(RuntimeError, match="divisible by 8"):
        torch.ops.mslk.f8f8bf16_rowwise_grouped_mm(XQ.view(2, 32, 512), WQ[:, :12].contiguous(), xs.view(2, 32),
                                                   ws[:, :12].contiguous(), None,
                                                   torch.empty(2, 32, 12, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(RuntimeError, match="3 dimensions"):
        torch.ops.mslk.f8f8bf16_rowwise_batched(XQ, WQ, xs, ws)
    with pytest.raises(RuntimeError, match="use_fast_accum"):
        torch.ops.mslk.f8f8bf16_rowwise_batched(XQ.view(2, 32, 512), WQ, xs.view(2, 32), ws, None, False)
    # empty output: returned as is
    e = torch.ops.mslk.f8f8bf16_rowwise_grouped_mm(XQ[:0], WQ, xs[:0], ws, torch.zeros(2, dtype=torch.int32, device=DEV),
                                                   torch.empty(0, 512, dtype=torch.bfloat16, device=DEV))
    assert e.shape == (0, 512)


def test_graph_replay_follows_device_side_group_sizes():
    """The group extents are read on the device, so a captured graph must follow offsets / sizes that
    change between replays (test/gemm/gemm_test.py:652,776 capture these ops); every replay is compared
    with an eager call on the same extents, with eager work between the replays."""
    g = torch.Generator().manual_seed(41)
    G, N, K, total = 4, 512, 512, 700
    xq, xs = _quant(total, K, g)
    wq, ws = _quant(G * N, K, g, 0.02)
    XQ, WQ, XS, WS = xq.to(DEV), wq.view(G, N, K).to(DEV), xs.to(DEV), ws.view(G, N).to(DEV)
    ends = torch.zeros(G, dtype=torch.int32, device=DEV)
    sizes = torch.zeros(G, dtype=torch.int64, device=DEV)
    out = _sentinel(total, N)
    splits = [[100, 200, 300, 100], [0, 700, 0, 0], [1, 2, 3, 4], [175, 175, 175, 175]]

    def set_split(ms):
        ends.copy_(torch.tensor(ms, dtype=torch.int64).cumsum(0).to(torch.int32))
        sizes.copy_(torch.tensor(ms, dtype=torch.int64))

    set_split(splits[0])
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):   # warm-up outside capture
        torch.ops.mslk.f8f8bf16_rowwise_grouped_mm(XQ, WQ, XS, WS, ends, out)
        torch.ops.mslk.f8f8bf16_rowwise_grouped_stacked(XQ, WQ, XS, WS, sizes)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        torch.ops.mslk.f8f8bf16_rowwise_grouped_mm(XQ, WQ, XS, WS, ends, out)
        y_stacked = torch.ops.mslk.f8f8bf16_rowwise_grouped_stacked(XQ, WQ, XS, WS, sizes)
    for ms in splits:
        set_split(ms)
        out.fill_(SENTINEL)
        y_stacked.fill_(SENTINEL)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        eager = torch.ops.mslk.f8f8bf16_rowwise_grouped_mm(XQ, WQ, XS, WS, ends, _sentinel(total, N))   # eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(out, eager) and torch.equal(y_stacked, eager)
        r0 = 0
        for gi, m in enumerate(ms):
            if m:
                assert_gemm_close(out[r0:r0 + m], O.dequant_matmul(xq[r0:r0 + m], wq[gi * N:(gi + 1) * N], xs[r0:r0 + m],
                                                                   ws[gi * N:(gi + 1) * N]), f"split {ms} group {gi}")
            r0 += m
        assert (out[r0:] == SENTINEL).all()
