"""CPU-side checks of the boundary: the shared library loads, exports every symbol the header
declares, the operators are registered with the reference's schemas, and the shape functions and
argument checks behave like the reference's."""
import os
import re

import pytest
import torch

import mslk_amd
from mslk_amd import _lib, gemm

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F8 = torch.float8_e4m3fn


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "mslk_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mslk_amd_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = _lib.lib()
    names = _declared_symbols()
    assert len(names) >= 8
    for n in names:
        assert hasattr(L, n), f"{n} declared in include/mslk_amd.h but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert L.mslk_amd_version().decode().startswith("mslk_amd")
    assert L.mslk_amd_f8f8bf16_rowwise_workspace_bytes(4096, 4096, 4096) == 0
    assert L.mslk_amd_f8f8bf16_rowwise_workspace_bytes(128, 512, 14336) == 8 * 128 * 512 * 4      # eight K slices of fp32 sums
    assert L.mslk_amd_f8f8bf16_rowwise_workspace_bytes(64, 512, 8192) == 0                       # M <= 64 is not split below K = 12288


def test_c_abi_rejects_bad_arguments_without_a_gpu():
    L = _lib.lib()
    assert L.mslk_amd_quantize_fp8_row(None, 7, 1, 16, 16, None, 16, None, None, None) != 0
    assert b"dtype" in L.mslk_amd_last_error()
    assert L.mslk_amd_quantize_fp8_row(None, 0, 1, 16, 16, None, 8, None, None, None) != 0
    assert b"K_out" in L.mslk_amd_last_error()
    assert L.mslk_amd_f8f8bf16_rowwise(None, None, None, None, None, 0, None, -1, 4, 4, None, 0, None) != 0
    assert L.mslk_amd_f8f8bf16_rowwise(None, None, None, None, None, 2, None, 4, 4, 4, None, 0, None) != 0
    assert b"bias" in L.mslk_amd_last_error()
    assert L.mslk_amd_f8f8bf16_rowwise_grouped_mm(None, None, None, None, None, 9, 1, 4, 8, 16, None, None) != 0
    assert b"layout" in L.mslk_amd_last_error()
    assert L.mslk_amd_f8f8bf16_rowwise_grouped_mm(None, None, None, None, None, 1, 1, 4, 8, 16, None, None) != 0
    assert b"offsets are required" in L.mslk_amd_last_error()
    assert L.mslk_amd_f8f8bf16_rowwise_batched(None, None, None, None, None, 1, 2, 4, 8, 16, None, None) != 0
    assert b"bias" in L.mslk_amd_last_error()
    assert L.mslk_amd_f8f8bf16_rowwise_batched(None, None, None, None, None, 0, 0, 4, 8, 16, None, None) == 0
    assert L.mslk_amd_debug_tile_streams(None, 0, None, 0, 8192, 2, 128, 4, None) != 0
    assert b"which" in L.mslk_amd_last_error()
    assert L.mslk_amd_debug_tile_streams(None, 0, None, 0, 100, 2, 128, 3, None) != 0
    assert b"multiple of 128" in L.mslk_amd_last_error()
    assert L.mslk_amd_debug_tile_streams(None, 2 * 128 * 256 - 1, None, 128 * 64 * 256, 256, 2, 128, 3, None) != 0
    assert b"must hold" in L.mslk_amd_last_error()
    # empty problems are a successful no-op and touch no pointer
    assert L.mslk_amd_f8f8bf16_rowwise(None, None, None, None, None, 0, None, 0, 4, 4, None, 0, None) == 0
    assert L.mslk_amd_quantize_fp8_row(None, 0, 0, 16, 16, None, 16, None, None, None) == 0


@pytest.mark.parametrize("M,N,K,slices", [
    (64, 512, 8192, 0), (65, 512, 8192, 8),              # more than 64 rows: below, the weight-streaming kernel covers the CUs ...
    (32, 512, 14336, 0), (33, 512, 14336, 8), (64, 4096, 12288, 4), (64, 4096, 11008, 0),   # ... except 33 - 64 rows at K >= 12288
    (128, 512, 8192, 8), (128, 512, 6144, 6),            # as many slices as fill the CUs once, at least eight K steps each
    (128, 512, 4096, 0),                                 # K too short for two launches to pay
    (128, 4096, 8192, 2), (128, 4096, 6144, 0),          # half the CUs covered: from K = 8192 on
    (128, 4160, 8192, 0), (512, 1024, 8192, 2), (512, 1088, 8192, 0), (1024, 512, 16384, 2), (1025, 512, 16384, 0),   # at most 128 tiles of 64 x 64
    (96, 2048, 8192, 4), (300, 518, 6160, 5), (128, 63, 8192, 0),
])
def test_k_split_plan_is_pinned(M, N, K, slices):
    """mslk_amd_f8f8bf16_rowwise_workspace_bytes is the plan: slices * M * N floats for a shape the library splits along K
    (on a whole MI355X, which is also what the library assumes when no device can be queried), 0 otherwise."""
    assert _lib.lib().mslk_amd_f8f8bf16_rowwise_workspace_bytes(M, N, K) == slices * M * N * 4


def test_ops_registered_with_reference_schemas():
    s = str(torch.ops.mslk.f8f8bf16_rowwise.default._schema)
    assert s == ("mslk::f8f8bf16_rowwise(Tensor XQ, Tensor WQ, Tensor x_scale, Tensor w_scale, "
                 "Tensor? bias=None, bool use_fast_accum=True) -> Tensor")
    s = str(torch.ops.mslk.f8f8bf16_rowwise_out.default._schema)
    assert "Tensor(a!) output, Tensor? bias=None, bool use_fast_accum=True) -> ()" in s
    s = str(torch.ops.mslk.f8f8bf16_rowwise_grouped.default._schema)
    assert s == "mslk::f8f8bf16_rowwise_grouped(Tensor[] XQ, Tensor[] WQ, Tensor[] x_scale, Tensor[] w_scale) -> Tensor[]"
    s = str(torch.ops.mslk.f8f8bf16_rowwise_grouped_stacked.default._schema)
    assert s.endswith("(Tensor XQ, Tensor WQ, Tensor x_scale, Tensor w_scale, Tensor M_sizes) -> Tensor")
    s = str(torch.ops.mslk.f8f8bf16_rowwise_grouped_mm.default._schema)
    assert s == ("mslk::f8f8bf16_rowwise_grouped_mm(Tensor XQ, Tensor WQ, Tensor x_scale, Tensor w_scale, "
                 "Tensor? offsets, Tensor(a!) output) -> Tensor")
    s = str(torch.ops.mslk.f8f8bf16_rowwise_batched.default._schema)
    assert s == ("mslk::f8f8bf16_rowwise_batched(Tensor XQ, Tensor WQ, Tensor x_scale, Tensor w_scale, "
                 "Tensor? bias=None, bool use_fast_accum=True, Tensor(a!)? output=None) -> Tensor")
    s = str(torch.ops.mslk.f8f8f16_rowwise.default._schema)
    assert s == ("mslk::f8f8f16_rowwise(Tensor XQ, Tensor WQ, Tensor x_scale, Tensor w_scale, "
                 "Tensor? bias=None, bool use_fast_accum=True) -> Tensor")
    s = str(torch.ops.mslk.f8f8bf16_rowwise_grouped_dynamic.default._schema)
    assert s.endswith("Tensor zero_start_index_M, bool zeroing_output_tensor=True) -> Tensor")
    assert hasattr(torch.ops.mslk, "dequantize_fp8_row")
    # the quantizer under the names callers of the reference use (mslk/quantize/triton/fp8_quantize.py:319-328)
    s = str(torch.ops.triton.quantize_fp8_row.default._schema)
    assert s == ("triton::quantize_fp8_row(Tensor a, Tensor? scale_ub=None, Tensor? zero_start_index_M=None, "
                 "bool use_triton=True, Device? output_device=None, SymInt? align_rows_to=None, "
                 "float? eps_opt=0.001953125) -> (Tensor, Tensor)")
    s = str(torch.ops.mslk.quantize_fp8_per_row.default._schema)
    assert s == ("mslk::quantize_fp8_per_row(Tensor input, Tensor? bs=None, Tensor? scale_ub=None, "
                 "ScalarType? output_dtype=None, bool stochastic_rounding=False) -> (Tensor, Tensor)")


def test_fake_kernels_give_reference_shapes():
    from torch._subclasses.fake_tensor import FakeTensorMode
    with FakeTensorMode():
        dev = "cuda"
        wq = torch.empty(256, 128, dtype=F8, device=dev)
        y = torch.ops.mslk.f8f8bf16_rowwise(torch.empty(64, 128, dtype=F8, device=dev), wq,
                                            torch.empty(64, device=dev), torch.empty(256, device=dev))
        assert y.shape == (64, 256) and y.dtype == torch.bfloat16
        y = torch.ops.mslk.f8f8bf16_rowwise(torch.empty(3, 64, 128, dtype=F8, device=dev), wq,
                                            torch.empty(3, 64, device=dev), torch.empty(256, device=dev))
        assert y.shape == (3, 64, 256)
        ys = torch.ops.mslk.f8f8bf16_rowwise_grouped(
            [torch.empty(5, 512, dtype=F8, device=dev), torch.empty(0, 512, dtype=F8, device=dev)],
            [torch.empty(512, 512, dtype=F8, device=dev)] * 2,
            [torch.empty(5, device=dev), torch.empty(0, device=dev)], [torch.empty(512, device=dev)] * 2)
        assert [tuple(t.shape) for t in ys] == [(5, 512), (0, 512)]
        y = torch.ops.mslk.f8f8bf16_rowwise_grouped_stacked(
            torch.empty(40, 512, dtype=F8, device=dev), torch.empty(4, 768, 512, dtype=F8, device=dev),
            torch.empty(40, device=dev), torch.empty(4, 768, device=dev), torch.empty(4, dtype=torch.int64, device=dev))
        assert y.shape == (40, 768)
        out = torch.empty(40, 768, dtype=torch.bfloat16, device=dev)
        y = torch.ops.mslk.f8f8bf16_rowwise_grouped_mm(
            torch.empty(40, 512, dtype=F8, device=dev), torch.empty(4, 768, 512, dtype=F8, device=dev),
            torch.empty(40, device=dev), torch.empty(4, 768, device=dev), torch.empty(4, dtype=torch.int32, device=dev), out)
        assert y.shape == (40, 768)
        y = torch.ops.mslk.f8f8bf16_rowwise_batched(
            torch.empty(3, 40, 512, dtype=F8, device=dev), torch.empty(3, 768, 512, dtype=F8, device=dev),
            torch.empty(3, 40, device=dev), torch.empty(3, 768, device=dev))
        assert y.shape == (3, 40, 768) and y.dtype == torch.bfloat16
        q, s = torch.ops.triton.quantize_fp8_row(torch.empty(2, 3, 100, dtype=torch.bfloat16, device=dev), align_rows_to=16)
        assert q.shape == (2, 3, 112) and q.dtype == F8 and s.shape == (2, 3) and s.dtype == torch.float32
        q, s = torch.ops.mslk.quantize_fp8_per_row(torch.empty(5, 100, dtype=torch.float16, device=dev))
        assert q.shape == (5, 100) and q.dtype == F8 and s.shape == (5,) and s.dtype == torch.float32


def test_argument_checks_raise_like_the_reference():
    xq = torch.zeros(4, 32).to(F8)
    wq = torch.zeros(8, 32).to(F8)
    xs, ws = torch.ones(4), torch.ones(8)
    with pytest.raises(RuntimeError, match="dtypes must match"):
        gemm._rowwise_impl(xq, wq.view(torch.uint8), xs, ws, None, True)
    with pytest.raises(RuntimeError, match="Scales must be float32"):
        gemm._rowwise_impl(xq, wq, xs.double(), ws, None, True)
    with pytest.raises(RuntimeError, match="use_fast_accum"):
        gemm._rowwise_impl(xq, wq, xs, ws, None, False)
    with pytest.raises(RuntimeError, match="same number of groups"):
        gemm._check_grouped([xq], [wq, wq], [xs], [ws])
    with pytest.raises(RuntimeError):
        mslk_amd.quantize_fp8_row(torch.zeros(4, 4, dtype=torch.bfloat16))  # CPU tensor: no CPU implementation
    with pytest.raises(NotImplementedError):
        torch.ops.mslk.f8f8bf16_rowwise(xq, wq, xs, ws)  # no CPU kernel is registered


def test_product_package_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "mslk_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "import oracle" not in text and "from oracle" not in text and "liboracle" not in text, f


# (M, N, K, bias code, y dtype code, pre-shuffled, with workspace) -> the kernel the dense entry points pick on a whole
# MI355X.  The thresholds behind these choices were measured; an edit that moves one of the benchmark configurations (or
# a neighbouring shape class) to another kernel has to change this table knowingly.
DISPATCH_TABLE = [
    ((1024, 1024, 1024, 0, 0, 0, 1), "dense_tiled<64,64,waves=4x1,ring=5> tiles=256"),                       # cfg0
    ((4096, 4096, 4096, 0, 0, 0, 1), "dense_tiled<256,256,waves=2x2,ring=0> tiles=256"),                     # cfg1
    ((8192, 28672, 4096, 2, 0, 0, 1), "dense_persistent<256,256> tiles=3584 workgroups=256"),                # cfg2
    ((1, 8192, 8192, 0, 0, 0, 1), "skinny_lds<m_frags=1,n_frags=1,steps=4> workgroups=512"),                 # cfg3, M = 1
    ((4, 8192, 8192, 0, 0, 0, 1), "skinny_lds<m_frags=1,n_frags=1,steps=4> workgroups=512"),
    ((16, 8192, 8192, 0, 0, 0, 1), "dense_tiled<32,32,waves=2x1,ring=8> weights streamed tiles=256"),
    ((64, 8192, 8192, 0, 0, 0, 1), "dense_tiled<64,32,waves=4x1,ring=6> weights streamed tiles=256"),
    ((16, 8192, 8192, 0, 0, 1, 1), "skinny_lds<m_frags=1,n_frags=2,steps=2> preshuffled workgroups=256"),    # cfg3 on blocked weights
    ((64, 8192, 8192, 0, 0, 1, 1), "skinny_lds<m_frags=4,n_frags=2,steps=1> preshuffled workgroups=256"),
    ((64, 4096, 14336, 0, 0, 0, 0), "skinny_lds<m_frags=4,n_frags=1,steps=1> workgroups=256"),
    ((64, 4096, 14336, 0, 0, 0, 1), "splitk_partial<64,64,waves=4x1,ring=5> slices=4 + splitk_reduce"),       # 33 - 64 rows: split from K = 12288 on, given a workspace
    ((8, 8192, 8192, 0, 0, 0, 1), "skinny_lds<m_frags=1,n_frags=1,steps=4> workgroups=512"),                  # last M of the streaming kernel on wide weights
    ((9, 8192, 8192, 0, 0, 0, 1), "dense_tiled<32,32,waves=2x1,ring=8> weights streamed tiles=256"),
    ((32, 10240, 8192, 0, 0, 0, 1), "dense_tiled<64,64,waves=4x1,ring=5> weights streamed tiles=160"),        # M <= 32 on wider weights
    ((9, 22016, 8192, 0, 0, 0, 1), "dense_tiled<64,32,waves=4x1,ring=6> weights streamed tiles=688"),
    ((32, 32768, 7168, 0, 0, 0, 1), "dense_tiled<64,64,waves=4x1,ring=5> weights streamed tiles=512"),
    ((3, 1000, 272, 0, 0, 0, 1), "skinny_registers<m_frags=1,n_frags=1,steps=8> workgroups=63"),              # K % 1024 != 0
    ((8192, 8192, 8192, 0, 0, 0, 1), "dense_persistent<256,256> tiles=1024 workgroups=256"),
    ((2304, 8192, 8192, 0, 0, 0, 1), "dense_tiled<256,256,waves=2x2,ring=0> tiles=256 + dense_tiled<128,64,waves=4x1,ring=6> tiles=256"),
    ((3328, 8192, 8192, 0, 0, 0, 1), "dense_tiled<256,256,waves=2x2,ring=0> tiles=256 + dense_tiled<192,256,waves=2x2,ring=0> tiles=224"),   # last pass 5/8 full: its rows on 192-row tiles
    ((3840, 8192, 8192, 0, 0, 0, 1), "dense_persistent<256,256> tiles=480 workgroups=256"),                  # 7/8 full: one persistent launch
    ((2048, 4096, 4096, 0, 0, 0, 1), "dense_tiled<128,256,waves=2x2,ring=3> tiles=256"),
    ((1536, 6144, 8192, 0, 0, 0, 1), "dense_tiled<192,256,waves=2x2,ring=0> tiles=192"),                     # 144 tiles of 256 x 256: 192-row tiles still fit one per CU
    ((1728, 8192, 8192, 0, 0, 0, 1), "dense_tiled<256,256,waves=2x2,ring=0> tiles=224"),                     # ... and here they do not
    ((1536, 6144, 1024, 0, 0, 0, 1), "dense_tiled<256,256,waves=2x2,ring=0> tiles=144"),                     # short K keeps the fused epilogue of the 256 x 256 tiles
    ((768, 7168, 6144, 0, 0, 0, 1), "dense_tiled<192,128,waves=2x2,ring=3> tiles=224"),
    ((128, 512, 14336, 0, 0, 0, 1), "splitk_partial<64,64,waves=4x1,ring=5> slices=8 + splitk_reduce"),       # few tiles, long K, workspace given
    ((128, 512, 14336, 0, 0, 0, 0), "dense_tiled<128,32,waves=4x1,ring=8> weights streamed tiles=16"),         # ... and not given
    ((128, 4096, 14336, 2, 1, 0, 1), "splitk_partial<64,64,waves=4x1,ring=5> slices=2 + splitk_reduce"),
    ((128, 4096, 4096, 0, 0, 0, 1), "dense_tiled<64,64,waves=4x1,ring=5> tiles=128"),                          # K too short to split                      # 128 x 128 tiles would need two passes
    ((512, 8192, 8192, 0, 0, 0, 1), "dense_tiled<128,128,waves=2x2,ring=5> tiles=256"),
    ((384, 8192, 8192, 0, 0, 0, 1), "dense_tiled<96,128,waves=2x2,ring=5> tiles=256"),                        # 96-row tiles still fit one per CU: 256 instead of 192 tiles
    ((256, 8192, 8192, 0, 0, 0, 1), "dense_tiled<128,64,waves=4x1,ring=6> tiles=256"),
    ((128, 8192, 8192, 0, 0, 0, 1), "dense_tiled<64,64,waves=4x1,ring=5> tiles=256"),
    ((64, 10240, 8192, 0, 0, 0, 1), "dense_tiled<64,64,waves=4x1,ring=5> weights streamed tiles=160"),         # one row of tiles: non-temporal weight loads
    ((128, 28672, 4096, 0, 0, 0, 1), "dense_tiled<128,128,waves=2x2,ring=5> weights streamed tiles=224"),
    ((100, 57344, 8192, 0, 0, 0, 1), "dense_tiled<128,256,waves=2x2,ring=3> weights streamed tiles=224"),
    ((4096, 8192, 4096, 0, 0, 0, 1), "dense_persistent<256,256> tiles=512 workgroups=256"),
    ((4096, 4096, 4096, 0, 1, 1, 1), "dense_tiled<256,256,waves=2x2,ring=0> preshuffled tiles=256"),
    ((4096, 4096, 4100, 0, 0, 0, 1), "pad_rows + pad_rows + dense_tiled<256,256,waves=2x2,ring=0> tiles=256"),
    ((4096, 4096, 4100, 0, 0, 0, 0), "generic_scalar"),
    ((5, 7, 0, 0, 0, 0, 1), "fill_zero"),
    ((0, 16, 16, 0, 0, 0, 1), "nothing to launch"),
]


@pytest.mark.parametrize("args,want", DISPATCH_TABLE)
def test_dispatch_of_the_dense_entry_points_is_pinned(args, want):
    """mslk_amd_debug_dispatch_name runs the real dispatch code as a dry run (nothing is launched, no GPU needed: without
    one it assumes the 256 compute units of a whole MI355X)."""
    from mslk_amd import _lib
    got = _lib.lib().mslk_amd_debug_dispatch_name(*args).decode()
    assert got == want


def test_dispatch_dry_run_reports_argument_errors_and_leaves_no_state():
    from mslk_amd import _lib
    L = _lib.lib()
    assert L.mslk_amd_debug_dispatch_name(16, 24, 64, 0, 0, 1, 1).decode().startswith("error: ")   # N % 16 != 0 for blocked weights
    assert L.mslk_amd_debug_dispatch_name(-1, 16, 16, 0, 0, 0, 1).decode().startswith("error: ")
    # the dry run is over when the call returns: a real call would launch again (here: rejected for its null output first)
    assert L.mslk_amd_f8f8bf16_rowwise(None, None, None, None, None, 0, None, 4, 4, 16, None, 0, None) != 0
