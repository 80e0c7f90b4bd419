"""GPU parity of the grouped (MoE) rowwise FP8 GEMMs: equal to a loop of dense calls and within the
north_star tolerance of the per-group oracle.  Cases follow test/gemm/gemm_test.py:603-856 and
test/gemm/triton/grouped_gemm_test.py:54-151."""
import pytest
import torch

import mslk_amd
from mslk_amd import workloads as W
from oracle import fp8_rowwise_oracle as O
from tests.helpers import assert_gemm_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F8 = torch.float8_e4m3fn


def _make_groups(ms, N, K, g):
    xq, wq, xs, ws = [], [], [], []
    for m in ms:
        x = torch.randn(m, K, generator=g).bfloat16()
        w = (torch.randn(N, K, generator=g) * 0.02).bfloat16()
        q, s = O.quantize_fp8_row(x) if m > 0 else (torch.empty(0, K, dtype=F8), torch.empty(0))
        xq.append(q); xs.append(s)
        q, s = O.quantize_fp8_row(w)
        wq.append(q); ws.append(s)
    return xq, wq, xs, ws


def _dev(ts):
    return [t.to(DEV) for t in ts]


@pytest.mark.parametrize("ms,N,K", [
    ([64], 512, 512), ([300, 0, 17, 256, 1], 768, 512), ([0, 0, 5], 512, 1024),
    ([128] * 16, 1024, 512), ([7, 300, 0, 0, 513, 64, 2, 1000], 520, 656),
    ([3] * 70, 512, 512),   # more groups than one launch carries in its argument block
    ([2100, 0, 5, 1030, 256, 257], 768, 512),   # groups cut into panels of four row tiles: row offsets inside a group
    ([1100] * 40, 512, 512),   # more panels than descriptors: the launch deals whole groups instead
])
def test_tensorlist_grouped(ms, N, K):
    g = torch.Generator().manual_seed(sum(ms) + N + K)
    xq, wq, xs, ws = _make_groups(ms, N, K, g)
    ys = torch.ops.mslk.f8f8bf16_rowwise_grouped(_dev(xq), _dev(wq), _dev(xs), _dev(ws))
    torch.cuda.synchronize()
    assert len(ys) == len(ms)
    refs = O.grouped_dequant_matmul(xq, wq, xs, ws)
    for m, y, r in zip(ms, ys, refs):
        assert y.shape == (m, N) and y.dtype == torch.bfloat16
        if m:
            assert_gemm_close(y, r)
    # outputs are views of one flat buffer, in group order
    base = ys[0].untyped_storage().data_ptr()
    assert all(y.untyped_storage().data_ptr() == base for y in ys)
    # concatenated variant
    ycat = torch.ops.mslk.f8f8bf16_rowwise_grouped_cat(_dev(xq), _dev(wq), _dev(xs), _dev(ws))
    torch.cuda.synchronize()
    assert torch.equal(ycat, torch.cat(ys, dim=0))


def test_grouped_equals_dense_loop_and_is_order_invariant():
    g = torch.Generator().manual_seed(31)
    ms = [300, 1, 640, 0, 77]
    xq, wq, xs, ws = _make_groups(ms, 768, 1024, g)
    dxq, dwq, dxs, dws = _dev(xq), _dev(wq), _dev(xs), _dev(ws)
    ys = torch.ops.mslk.f8f8bf16_rowwise_grouped(dxq, dwq, dxs, dws)
    order = [4, 2, 0, 3, 1]
    yp = torch.ops.mslk.f8f8bf16_rowwise_grouped([dxq[i] for i in order], [dwq[i] for i in order],
                                                 [dxs[i] for i in order], [dws[i] for i in order])
    torch.cuda.synchronize()
    for j, i in enumerate(order):
        assert torch.equal(yp[j], ys[i])
    for i, m in enumerate(ms):
        if m > 64:  # same tile kernel as the dense op above the skinny threshold: bitwise equal
            d = torch.ops.mslk.f8f8bf16_rowwise(dxq[i], dwq[i], dxs[i], dws[i])
            assert_gemm_close(ys[i], d.float().cpu())


def test_grouped_rejects_small_n_k_like_the_reference():
    g = torch.Generator().manual_seed(32)
    xq, wq, xs, ws = _make_groups([8], 256, 512, g)
    with pytest.raises(RuntimeError, match="at least 512"):
        torch.ops.mslk.f8f8bf16_rowwise_grouped(_dev(xq), _dev(wq), _dev(xs), _dev(ws))


@pytest.mark.parametrize("ms,N,K", [([64, 0, 300, 5], 512, 512), ([1] * 16, 768, 1024), ([0, 0, 0, 700], 520, 272),
                                    ([9, 40], 136, 200)])   # K not a multiple of 16: scalar tile path
def test_stacked_grouped(ms, N, K):
    g = torch.Generator().manual_seed(33)
    xq, wq, xs, ws = _make_groups(ms, N, K, g)
    XQ = torch.cat(xq).to(DEV)
    WQ = torch.stack(wq).to(DEV)
    XS = torch.cat(xs).to(DEV)
    WS = torch.stack(ws).to(DEV)
    msz = torch.tensor(ms, dtype=torch.int64, device=DEV)
    y = torch.ops.mslk.f8f8bf16_rowwise_grouped_stacked(XQ, WQ, XS, WS, msz)
    torch.cuda.synchronize()
    assert y.shape == (sum(ms), N)
    refs = [r for r, m in zip(O.grouped_dequant_matmul(xq, wq, xs, ws), ms) if m]
    assert_gemm_close(y, torch.cat(refs))


def test_cfg4_full():
    g = torch.Generator().manual_seed(104)
    wl = W.cfg4()
    assert sum(wl.counts) == 8192 and len(wl.counts) == 16
    xq_all, xs_all = mslk_amd.quantize_fp8_row(wl.x.to(DEV), use_triton=False)
    rq, rs = O.quantize_fp8_row(wl.x)
    assert torch.equal(xq_all.cpu().view(torch.uint8), rq.view(torch.uint8)) and torch.equal(xs_all.cpu().view(torch.int32), rs.view(torch.int32))
    wq, ws = [], []
    for w in wl.w:
        q, s = mslk_amd.quantize_fp8_row(w.to(DEV), use_triton=False)
        wq.append(q); ws.append(s)
    xq = list(xq_all.split(wl.counts)); xs = list(xs_all.split(wl.counts))
    ys = torch.ops.mslk.f8f8bf16_rowwise_grouped(xq, wq, xs, ws)
    torch.cuda.synchronize()
    assert sum(y.shape[0] for y in ys) == 8192
    # every row of every expert against the fp32 oracle (0.69 TFLOP of CPU work): the ragged last tile of each expert,
    # its last row and the tile edges of the large experts included
    for e, y in enumerate(ys):
        m = wl.counts[e]
        assert y.shape == (m, 8192)
        if m == 0:
            continue
        ref = O.dequant_matmul(xq[e].cpu(), wq[e].cpu(), xs[e].cpu(), ws[e].cpu())
        assert_gemm_close(y, ref, f"cfg4 expert {e} ({m} rows)")
    # stacked entry point on the same data gives the same bits
    y2 = torch.ops.mslk.f8f8bf16_rowwise_grouped_stacked(xq_all, torch.stack(wq), xs_all, torch.stack(ws),
                                                         torch.tensor(wl.counts, dtype=torch.int64, device=DEV))
    torch.cuda.synchronize()
    assert torch.equal(y2, torch.cat(ys))
