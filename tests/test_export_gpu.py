"""torch.export of the operators of the path: a small module is exported (strict, fake tensors), the exported program is
run on the GPU and must return what eager returns, bit for bit.
Reference: test/gemm/gemm_test.py:236-303 (ExportCompileTests: export of a module that calls f8f8bf16_rowwise, compile of
the rowwise ops), test/quantize/fp8_quantize_export_test.py:33-65 (eager vs compiled vs exported quantize_fp8_row)."""
import pytest
import torch

import mslk_amd

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F8 = torch.float8_e4m3fn


def _codes(*shape, seed=0):
    g = torch.Generator().manual_seed(seed + sum(shape))
    return (torch.randn(*shape, generator=g) * 2).to(F8).to(DEV)


def _same(a, b):
    if isinstance(a, (tuple, list)):
        assert len(a) == len(b)
        for x, y in zip(a, b):
            _same(x, y)
        return
    assert a.dtype == b.dtype and a.shape == b.shape
    assert torch.equal(a.view(torch.uint8) if a.dtype == F8 else a, b.view(torch.uint8) if b.dtype == F8 else b)


def _export_and_compare(mod, args, ops_expected):
    eager = mod(*args)
    ep = torch.export.export(mod, args, strict=True)
    targets = {str(n.target) for n in ep.graph.nodes if n.op == "call_function"}
    for name in ops_expected:
        assert any(name in t for t in targets), f"{name} is not a node of the exported graph: {sorted(targets)}"
    got = ep.module()(*args)
    torch.cuda.synchronize()
    _same(got, eager)
    return ep


def test_export_f8f8bf16_rowwise():
    class M(torch.nn.Module):
        def forward(self, xq, wq, xs, ws, bias):
            return torch.ops.mslk.f8f8bf16_rowwise(xq, wq, xs, ws, bias=bias), torch.ops.mslk.f8f8f16_rowwise(xq, wq, xs, ws)

    m, n, k = 256, 256, 256   # the reference's export shape
    args = (_codes(m, k), _codes(n, k, seed=1), torch.rand(m, device=DEV) + 0.5, torch.rand(n, device=DEV) + 0.5,
            torch.randn(n, device=DEV))
    _export_and_compare(M(), args, ["mslk.f8f8bf16_rowwise", "mslk.f8f8f16_rowwise"])


def test_export_f8f8bf16_rowwise_out():
    class M(torch.nn.Module):
        def forward(self, xq, wq, xs, ws):
            out = torch.empty(xq.shape[0], wq.shape[0], dtype=torch.bfloat16, device=xq.device)
            torch.ops.mslk.f8f8bf16_rowwise_out(xq, wq, xs, ws, out)
            return out

    m, n, k = 48, 520, 384
    args = (_codes(m, k), _codes(n, k, seed=1), torch.rand(m, device=DEV) + 0.5, torch.rand(n, device=DEV) + 0.5)
    _export_and_compare(M(), args, ["mslk.f8f8bf16_rowwise_out"])


def test_export_grouped_stacked_and_grouped_mm():
    class M(torch.nn.Module):
        def forward(self, xq, wq, xs, ws, sizes, ends):
            a = torch.ops.mslk.f8f8bf16_rowwise_grouped_stacked(xq, wq, xs, ws, sizes)
            out = torch.zeros(xq.shape[0], wq.shape[1], dtype=torch.bfloat16, device=xq.device)
            b = torch.ops.mslk.f8f8bf16_rowwise_grouped_mm(xq, wq, xs, ws, ends, out)
            return a, b

    ms = [5, 0, 300, 79]
    G, N, K, total = len(ms), 512, 512, sum(ms)
    sizes = torch.tensor(ms, dtype=torch.int64, device=DEV)
    args = (_codes(total, K), _codes(G, N, K, seed=1), torch.rand(total, device=DEV) + 0.5, torch.rand(G, N, device=DEV) + 0.5,
            sizes, sizes.cumsum(0).to(torch.int32))
    ep = _export_and_compare(M(), args, ["mslk.f8f8bf16_rowwise_grouped_stacked", "mslk.f8f8bf16_rowwise_grouped_mm"])
    # the group sizes are read on the device: the exported program follows new sizes without re-export
    ms2 = [100, 200, 0, 84]
    sizes2 = torch.tensor(ms2, dtype=torch.int64, device=DEV)
    args2 = args[:4] + (sizes2, sizes2.cumsum(0).to(torch.int32))
    _same(ep.module()(*args2), M()(*args2))


@pytest.mark.parametrize("align", [None, 16])
def test_export_quantize_fp8_row(align):
    class M(torch.nn.Module):
        def forward(self, x):
            return torch.ops.triton.quantize_fp8_row(x, align_rows_to=align)

    x = torch.randn(32, 40, device=DEV, dtype=torch.bfloat16)   # 40 columns: align_rows_to = 16 pads to 48
    ep = _export_and_compare(M(), (x,), ["triton.quantize_fp8_row"])
    q, s = ep.module()(x)
    assert q.shape == (32, 48 if align else 40) and s.shape == (32,)
    # and the Python wrapper, as the reference's export test calls it (eager == compiled == exported)
    class W(torch.nn.Module):
        def forward(self, x):
            return mslk_amd.quantize_fp8_row(x)

    eager = W()(x)
    _same(torch.compile(W(), backend="aot_eager")(x), eager)
    _same(torch.export.export(W(), (x,)).module()(x), eager)


def test_export_quantize_f8f8bf16_rowwise_and_the_linear_pair():
    class Fused(torch.nn.Module):
        def forward(self, x, wq, ws):
            return torch.ops.mslk.quantize_f8f8bf16_rowwise(x, wq, ws)

    class Pair(torch.nn.Module):
        def forward(self, x, wq, ws):
            xq, xs = torch.ops.triton.quantize_fp8_row(x, use_triton=False)
            return torch.ops.mslk.f8f8bf16_rowwise(xq, wq, xs, ws), xq, xs

    wq, ws = mslk_amd.quantize_fp8_row((torch.randn(520, 1024, device=DEV) * 0.02).bfloat16(), use_triton=False)
    for rows in (2, 40):   # one launch / two launches behind the same operator
        x = torch.randn(rows, 1024, device=DEV, dtype=torch.bfloat16)
        _export_and_compare(Fused(), (x, wq, ws), ["mslk.quantize_f8f8bf16_rowwise"])
        _export_and_compare(Pair(), (x, wq, ws), ["triton.quantize_fp8_row", "mslk.f8f8bf16_rowwise"])
        _same(Fused()(x, wq, ws), Pair()(x, wq, ws))
