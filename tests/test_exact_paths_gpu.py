"""Bit-exact GPU tests of the tile paths whose correctness rests on hand-counted hardware hazards.

The K loop and the epilogue of the LDS-tiled GEMM contain statements the compiler's hazard pass cannot see into (the
output store written as an instruction, explicit accumulator-register reads behind a fixed number of wait states, the
hand-computed load counter of the barrier).  A mistake there corrupts single values, rows or 8-byte pieces, usually by
small amounts: a tolerance against the fp32 oracle is the wrong net.  Here every input is an integer code in [-8, 8] with
power-of-two scales and small integer biases, so fp32 accumulation is exact in any order and the output must equal the
CPU result bit for bit.  One case per path: persistent workgroups (with the split-off last pass), the grouped kernels in
every row-skipping class and every device-extent layout (also with more than 64 and more than 128 groups), the batched op
with bias, and the pre-shuffled tiles.
Reference pattern: test/gemm/gemm_test.py:440-447,706-716,823-830 (equality of captured replays), 603-856 (grouped cases).
"""
import pytest
import torch

import mslk_amd

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F8 = torch.float8_e4m3fn
SENTINEL = -7.0


def _ints(rows, K, g):
    return torch.randint(-8, 9, (rows, K), generator=g).float()


def _pow2(n, g, lo=-3, hi=4):
    return 2.0 ** torch.randint(lo, hi, (n,), generator=g).float()


def _want(xi, wi, xs, ws, bias=None, fp16=False):
    v = (xi @ wi.T) * xs[:, None] * ws[None, :]
    if bias is not None:
        v = v + bias[None, :]
    return v.half() if fp16 else v.bfloat16()


def _same_bits(got, want, what):
    got = got.cpu()
    assert got.shape == want.shape and got.dtype == want.dtype, what
    bad = got.view(torch.int16) != want.view(torch.int16)
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.numel()} outputs differ, first at {bad.nonzero()[0].tolist()}"


@pytest.mark.parametrize("fp16_out", [False, True])
@pytest.mark.parametrize("bias_dtype", [None, torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [
    (4352, 4352, 384),    # 289 full tiles on 256 persistent workgroups: a second, short pass
    (4400, 4500, 272),    # ragged last rows and columns, a K tail
    (2304, 8192, 256),    # last pass less than half full: its rows go to a second launch with smaller tiles
    (8192, 4096, 128),    # 512 tiles, a K loop of one step
])
def test_persistent_workgroups_exact(M, N, K, bias_dtype, fp16_out):
    assert ((M + 255) // 256) * ((N + 255) // 256) > 256
    g = torch.Generator().manual_seed(M + 3 * N + K)
    xi, wi, xs, ws = _ints(M, K, g), _ints(N, K, g), _pow2(M, g), _pow2(N, g)
    bias = None if bias_dtype is None else torch.randint(-4, 5, (N,), generator=g).float()
    op = torch.ops.mslk.f8f8f16_rowwise if fp16_out else torch.ops.mslk.f8f8bf16_rowwise
    y = op(xi.to(F8).to(DEV), wi.to(F8).to(DEV), xs.to(DEV), ws.to(DEV), bias=None if bias is None else bias.to(bias_dtype).to(DEV))
    torch.cuda.synchronize()
    _same_bits(y, _want(xi, wi, xs, ws, bias, fp16_out), f"{M}x{N}x{K} bias={bias_dtype} fp16={fp16_out}")


# Row counts of the ragged last tile of a group in each class of the 256-row tile (<= 64, <= 128, <= 192, > 192 rows),
# whole tiles in front of a ragged one, a group of more than four row tiles (cut into panels), single rows, empty groups.
ROWSKIP_256 = [40, 0, 100, 180, 250, 256 + 64, 512 + 128, 1, 1024 + 192 + 1, 2100, 64, 65, 128, 129, 192, 193]
# the same for the 128-row tile (classes of 32 rows)
ROWSKIP_128 = [20, 0, 50, 90, 120, 128 + 10, 256 + 40, 1, 128 + 70, 384 + 100, 32, 33, 64, 65, 96, 97]


def _groups(ms, N, K, g):
    xi = [_ints(m, K, g) for m in ms]
    wi = [_ints(N, K, g) for _ in ms]
    xs = [_pow2(m, g) for m in ms]
    ws = [_pow2(N, g) for _ in ms]
    return xi, wi, xs, ws


@pytest.mark.parametrize("ms,N,K", [(ROWSKIP_256, 768, 640), (ROWSKIP_256[:9], 1024, 528), ([3] * 70, 512, 512),
                                    ([1100], 2304, 512), ([2100, 300], 1024, 640), ([257, 0, 1025], 4096, 512)])
def test_tensorlist_grouped_exact(ms, N, K):
    """grouped_tiled_kernel: 256 x 256 tiles, reduced K loops (1/4, 1/2, 3/4 of the m fragments) with the fragments dealt
    to the wave rows round-robin, panels of four row tiles, a K tail in the second case, more than 64 groups in the third;
    one to three groups in the others: fewer panels than XCDs, so the launcher cuts panels between XCDs."""
    g = torch.Generator().manual_seed(sum(ms) + N + K)
    xi, wi, xs, ws = _groups(ms, N, K, g)
    dev = lambda ts, f8=False: [(t.to(F8) if f8 else t).to(DEV) for t in ts]
    ys = torch.ops.mslk.f8f8bf16_rowwise_grouped(dev(xi, True), dev(wi, True), dev(xs), dev(ws))
    torch.cuda.synchronize()
    for e, m in enumerate(ms):
        assert ys[e].shape == (m, N)
        if m:
            _same_bits(ys[e], _want(xi[e], wi[e], xs[e], ws[e]), f"group {e} ({m} rows)")


@pytest.mark.parametrize("K", [128, 256, 384])
def test_tensorlist_grouped_exact_on_k_loops_of_one_two_and_three_steps(K):
    """The operator refuses K < 512 as the reference does (fp8_rowwise_grouped_gemm.hip:505-507); the C ABI does not, and the
    start and the end of the software pipeline of the K loop are exactly what such short loops consist of."""
    import ctypes
    from mslk_amd import _lib
    ms, N = [m for m in ROWSKIP_256 if m], 512
    g = torch.Generator().manual_seed(sum(ms) + N + K)
    xi, wi, xs, ws = _groups(ms, N, K, g)
    xq, wq = [t.to(F8).to(DEV) for t in xi], [t.to(F8).to(DEV) for t in wi]
    xsd, wsd = [t.to(DEV) for t in xs], [t.to(DEV) for t in ws]
    ys = [torch.full((m, N), SENTINEL, dtype=torch.bfloat16, device=DEV) for m in ms]
    G = len(ms)
    P, I = ctypes.c_void_p * G, ctypes.c_int64 * G
    ptrs = lambda ts: P(*[t.data_ptr() for t in ts])
    _lib.check(_lib.lib().mslk_amd_f8f8bf16_rowwise_grouped(G, ptrs(xq), ptrs(wq), ptrs(xsd), ptrs(wsd), ptrs(ys), I(*ms), I(*[N] * G),
                                                            I(*[K] * G), torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    for e, m in enumerate(ms):
        _same_bits(ys[e], _want(xi[e], wi[e], xs[e], ws[e]), f"group {e} ({m} rows)")


def _stacked_case(ms, N, K, g, extra=0):
    G, total = len(ms), sum(ms) + extra
    xi, wi = _ints(total, K, g), _ints(G * N, K, g)
    xs, ws = _pow2(total, g), _pow2(G * N, g)
    want = torch.full((total, N), SENTINEL, dtype=torch.bfloat16)
    r0 = 0
    for gi, m in enumerate(ms):
        if m:
            want[r0:r0 + m] = _want(xi[r0:r0 + m], wi[gi * N:(gi + 1) * N], xs[r0:r0 + m], ws[gi * N:(gi + 1) * N])
        r0 += m
    dev = (xi.to(F8).to(DEV), wi.to(F8).view(G, N, K).to(DEV), xs.to(DEV), ws.view(G, N).to(DEV))
    return dev, want, total


MANY_70 = [((i * 37) % 150 if i % 5 else 0) + (300 if i % 17 == 3 else 0) for i in range(70)]      # empty, ragged, multi-tile
MANY_130 = [((i * 53) % 97 if i % 4 else 0) + (260 if i % 31 == 7 else 0) for i in range(130)]


@pytest.mark.parametrize("ms,N,K,extra", [
    ([1024 + 40, 1024 + 100, 1024 + 180, 1024 + 250], 2560, 512, 0),   # average group large enough for 256 x 256 tiles
    (ROWSKIP_128, 512, 656, 5),                                        # 128 x 128 tiles, every row-skipping class, a K tail
    (MANY_70, 512, 512, 9),                                            # more than 64 groups: a second chunk of extents
    (MANY_130, 520, 528, 0),                                           # more than 128: a third; N % 256 != 0
    ([1024 + 40, 1024 + 100, 1024 + 180, 1024 + 250], 512, 256, 0),     # 256 x 256 tiles, K loops of two and of three steps
    ([1024 + 40, 1024 + 100, 1024 + 180, 1024 + 250], 512, 384, 3),
    (ROWSKIP_128, 512, 256, 0),                                        # the same on 128 x 128 tiles
])
def test_stacked_and_offsets_over_m_exact(ms, N, K, extra):
    """grouped_device_kernel with int64 sizes (stacked) and int32 cumulative ends (2D-3D): the same bits from both, rows
    beyond the last group untouched."""
    g = torch.Generator().manual_seed(sum(ms) + N + K + len(ms))
    (XQ, WQ, XS, WS), want, total = _stacked_case(ms, N, K, g, extra)
    ends = torch.tensor(ms, dtype=torch.int64).cumsum(0).to(torch.int32).to(DEV)
    out = torch.full((total, N), SENTINEL, dtype=torch.bfloat16, device=DEV)
    torch.ops.mslk.f8f8bf16_rowwise_grouped_mm(XQ, WQ, XS, WS, ends, out)
    torch.cuda.synchronize()
    _same_bits(out, want, f"offsets over M, G={len(ms)}")
    if N >= 512 and K >= 512 and extra == 0:
        y = torch.ops.mslk.f8f8bf16_rowwise_grouped_stacked(XQ, WQ, XS, WS, torch.tensor(ms, dtype=torch.int64, device=DEV))
        torch.cuda.synchronize()
        _same_bits(y, want, f"stacked, G={len(ms)}")
    elif N >= 512 and K >= 512:
        # the stacked operator allocates its own output; call the library on a sentinel-filled one to see the rows beyond
        from mslk_amd import _lib
        out2 = torch.full((total, N), SENTINEL, dtype=torch.bfloat16, device=DEV)
        msz = torch.tensor(ms, dtype=torch.int64, device=DEV)
        _lib.check(_lib.lib().mslk_amd_f8f8bf16_rowwise_grouped_stacked(XQ.data_ptr(), WQ.data_ptr(), XS.data_ptr(), WS.data_ptr(),
                                                                        msz.data_ptr(), len(ms), total, N, K, out2.data_ptr(),
                                                                        torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        _same_bits(out2, want, f"stacked through the C ABI, G={len(ms)}")


@pytest.mark.parametrize("ns,M,K,extra", [
    ([256 + 40, 512, 8, 0, 200, 768 + 24], 300, 528, 16),
    ([((i * 29) % 90 + 8) // 8 * 8 if i % 6 else 0 for i in range(70)], 100, 512, 0),
    ([((i * 13) % 60 + 8) // 8 * 8 if i % 3 else 0 for i in range(130)], 70, 272, 24),
])
def test_offsets_over_n_exact(ns, M, K, extra):
    """3D-2D: groups are column blocks of the output; more than 64 and more than 128 groups walk further chunks."""
    g = torch.Generator().manual_seed(sum(ns) + M + K)
    G, total = len(ns), sum(ns) + extra
    xi, wi, xs, ws = _ints(G * M, K, g), _ints(total, K, g), _pow2(G * M, g), _pow2(total, g)
    want = torch.full((M, total), SENTINEL, dtype=torch.bfloat16)
    c0 = 0
    for gi, n in enumerate(ns):
        if n:
            want[:, c0:c0 + n] = _want(xi[gi * M:(gi + 1) * M], wi[c0:c0 + n], xs[gi * M:(gi + 1) * M], ws[c0:c0 + n])
        c0 += n
    out = torch.full((M, total), SENTINEL, dtype=torch.bfloat16, device=DEV)
    ends = torch.tensor(ns, dtype=torch.int64).cumsum(0).to(torch.int32).to(DEV)
    torch.ops.mslk.f8f8bf16_rowwise_grouped_mm(xi.to(F8).view(G, M, K).to(DEV), wi.to(F8).to(DEV), xs.view(G, M).to(DEV),
                                               ws.to(DEV), ends, out)
    torch.cuda.synchronize()
    _same_bits(out, want, f"offsets over N, G={G}")


@pytest.mark.parametrize("ks,M,N", [([512, 128, 0, 256, 48], 300, 520), ([1024, 2048], 1100, 1024)])
def test_offsets_over_k_exact(ks, M, N):
    """2D-2D: groups are K slices of both operands; an empty slice writes zeros."""
    g = torch.Generator().manual_seed(sum(ks) + M + N)
    G, total = len(ks), sum(ks)
    xi, wi, xs, ws = _ints(M, total, g), _ints(N, total, g), _pow2(G * M, g), _pow2(G * N, g)
    want = torch.empty(G, M, N, dtype=torch.bfloat16)
    k0 = 0
    for gi, k in enumerate(ks):
        want[gi] = _want(xi[:, k0:k0 + k], wi[:, k0:k0 + k], xs[gi * M:(gi + 1) * M], ws[gi * N:(gi + 1) * N])
        k0 += k
    out = torch.full((G, M, N), SENTINEL, dtype=torch.bfloat16, device=DEV)
    ends = torch.tensor(ks, dtype=torch.int64).cumsum(0).to(torch.int32).to(DEV)
    torch.ops.mslk.f8f8bf16_rowwise_grouped_mm(xi.to(F8).to(DEV), wi.to(F8).to(DEV), xs.to(DEV), ws.to(DEV), ends, out)
    torch.cuda.synchronize()
    _same_bits(out, want, "offsets over K")


@pytest.mark.parametrize("G,M,N,K,live", [(4, 300, 512, 512, [300, 0, 17, 256]), (3, 1100, 2048, 528, [513, 1100, 255]),
                                          (24, 512, 2304, 512, [(i * 61) % 513 for i in range(24)])])
def test_grouped_dynamic_exact(G, M, N, K, live):
    """Pre-padded groups: only the first live[g] rows of group g are multiplied; the rest reads as zero."""
    g = torch.Generator().manual_seed(G + M + N + K)
    xi, wi, xs, ws = _ints(G * M, K, g), _ints(G * N, K, g), _pow2(G * M, g), _pow2(G * N, g)
    y = torch.ops.mslk.f8f8bf16_rowwise_grouped_dynamic(xi.to(F8).view(G, M, K).to(DEV), wi.to(F8).view(G, N, K).to(DEV),
                                                        xs.view(G, M).to(DEV), ws.view(G, N).to(DEV),
                                                        torch.tensor(live, dtype=torch.int64, device=DEV))
    torch.cuda.synchronize()
    want = torch.zeros(G, M, N, dtype=torch.bfloat16)
    for gi, m in enumerate(live):
        rows, cols = slice(gi * M, gi * M + m), slice(gi * N, (gi + 1) * N)
        want[gi, :m] = _want(xi[rows], wi[cols], xs[rows], ws[cols])
    _same_bits(y, want, "dynamic")


@pytest.mark.parametrize("bias_dtype", [None, torch.float32, torch.bfloat16])
@pytest.mark.parametrize("G,M,N,K", [(16, 512, 768, 384), (5, 300, 1032, 528), (3, 1100, 2304, 256)])
def test_batched_exact(G, M, N, K, bias_dtype):
    """The uniform layout (3D-3D / batched), 128 x 128 and 256 x 256 tiles, with the per-batch bias [G, N]."""
    g = torch.Generator().manual_seed(G + M + N + K)
    xi, wi, xs, ws = _ints(G * M, K, g), _ints(G * N, K, g), _pow2(G * M, g), _pow2(G * N, g)
    bias = None if bias_dtype is None else torch.randint(-4, 5, (G, N), generator=g).float()
    y = torch.ops.mslk.f8f8bf16_rowwise_batched(xi.to(F8).view(G, M, K).to(DEV), wi.to(F8).view(G, N, K).to(DEV),
                                                xs.view(G, M).to(DEV), ws.view(G, N).to(DEV),
                                                None if bias is None else bias.to(bias_dtype).to(DEV))
    torch.cuda.synchronize()
    want = torch.stack([_want(xi[b * M:(b + 1) * M], wi[b * N:(b + 1) * N], xs[b * M:(b + 1) * M], ws[b * N:(b + 1) * N],
                              None if bias is None else bias[b]) for b in range(G)])
    _same_bits(y, want, f"batched bias={bias_dtype}")


@pytest.mark.parametrize("fp16_out", [False, True])
@pytest.mark.parametrize("M,N,K", [
    (3072, 3328, 384),    # 156 tiles of 256 x 256, one per workgroup (interior tiles: last K step under the epilogue)
    (4352, 4352, 256),    # persistent workgroups
    (1024, 4096, 320),    # 128 x 256 ring tiles; K tail of 64
    (512, 2048, 448),     # 128 x 128 ring
    (200, 2048, 512),     # 128 x 64 / 64 x 64 narrow tiles
    (48, 4096, 1024),     # weight-streaming kernel on blocked weights
    (40, 2560, 5504), (20, 8192, 11008),   # ... on K steps that do not divide among its waves
    (10, 2048, 2048), (30, 1024, 1024), (60, 4096, 1024), (60, 8192, 1024),   # 16 weight rows per workgroup up to N = 4096, 32 above
    (300, 8000, 448),     # 96 x 128 ring tiles
    (1000, 5008, 576),    # 192 x 128 tiles (ragged rows and columns; N % 16 == 0 and K % 64 == 0 as blocked weights need)
    (1500, 6096, 2112),   # 192 x 256 tiles
])
def test_preshuffled_tiles_exact(M, N, K, fp16_out):
    g = torch.Generator().manual_seed(M + N + K)
    xi, wi, xs, ws = _ints(M, K, g), _ints(N, K, g), _pow2(M, g), _pow2(N, g)
    bias = torch.randint(-4, 5, (N,), generator=g).float()
    wshuf = mslk_amd.preshuffle_b_mfma(wi.to(F8).to(DEV))
    op = torch.ops.mslk.f8f8f16_rowwise_preshuffle if fp16_out else torch.ops.mslk.f8f8bf16_rowwise_preshuffle
    for b in (None, bias):
        y = op(xi.to(F8).to(DEV), wshuf, xs.to(DEV), ws.to(DEV), bias=None if b is None else b.to(DEV))
        torch.cuda.synchronize()
        _same_bits(y, _want(xi, wi, xs, ws, b, fp16_out), f"pre-shuffled {M}x{N}x{K} bias={'yes' if b is not None else 'no'}")


def test_rows_of_a_partly_filled_last_pass_go_to_a_second_launch_exact():
    """416 tiles of 256 x 256 on 256 CUs: the 2048 rows of the first pass and the 1280 rows behind them are two launches
    (256 x 256 tiles, then 192 x 256 tiles); the seam between them must not show."""
    M, N, K = 3328, 8192, 2048
    g = torch.Generator().manual_seed(M + N + K)
    xi, wi, xs, ws = _ints(M, K, g), _ints(N, K, g), _pow2(M, g), _pow2(N, g)
    y = torch.ops.mslk.f8f8bf16_rowwise(xi.to(F8).to(DEV), wi.to(F8).to(DEV), xs.to(DEV), ws.to(DEV))
    torch.cuda.synchronize()
    _same_bits(y, _want(xi, wi, xs, ws), f"{M}x{N}x{K}")


@pytest.mark.parametrize("M,N,K", [(1024, 8192, 384), (2048, 4096, 272), (96, 8192, 512), (128, 4096, 400), (40, 8192, 1040),
                                   (24, 12288, 256), (16, 12288, 256), (24, 20480, 384), (64, 16384, 384), (1536, 6144, 144),
                                   (300, 8192, 528), (280, 8000, 400), (384, 8192, 256),        # 96 x 128 tiles, ring of five
                                   (1000, 5000, 528), (768, 7168, 256), (960, 6144, 128),       # 192 x 128 tiles, ring of three
                                   (1536, 6144, 2064), (1500, 6100, 2048)])                      # 192 x 256 tiles, two-plus-three buffers
def test_ring_and_short_tiles_exact(M, N, K):
    """The symmetric-ring tile shapes (128 x 256, 192 x 128, 128 x 128, 96 x 128, 128 x 64, 128 x 32, 64 x 64, 64 x 32, 32 x 32): their
    barrier waits on a load count that covers several steps in flight; and the 192 x 256 tiles (six m fragments per wave on
    the two-plus-three buffers).  Ragged last tiles along M and N, K loops shorter than the ring, K tails."""
    g = torch.Generator().manual_seed(M + N + K)
    xi, wi, xs, ws = _ints(M, K, g), _ints(N, K, g), _pow2(M, g), _pow2(N, g)
    bias = torch.randint(-4, 5, (N,), generator=g).float()
    y = torch.ops.mslk.f8f8bf16_rowwise(xi.to(F8).to(DEV), wi.to(F8).to(DEV), xs.to(DEV), ws.to(DEV), bias=bias.bfloat16().to(DEV))
    torch.cuda.synchronize()
    _same_bits(y, _want(xi, wi, xs, ws, bias), f"{M}x{N}x{K}")


@pytest.mark.parametrize("fp16_out", [False, True])
@pytest.mark.parametrize("bias_dtype", [None, torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(128, 512, 8192), (96, 2048, 8192), (300, 518, 6160), (65, 4096, 14336), (512, 1024, 8208), (40, 1000, 12304)])
def test_k_split_exact(M, N, K, bias_dtype, fp16_out):
    """Few output tiles and a long K: with the workspace the library asks for, K is cut into slices whose fp32 sums a
    second launch adds, scales and converts (ragged rows and columns, a column count that rules out 16-byte accesses, a K
    tail in the last slice).  Same bits as the product of the codes, and as the unsplit kernels give without a workspace."""
    from mslk_amd import _lib
    L = _lib.lib()
    need = L.mslk_amd_f8f8bf16_rowwise_workspace_bytes(M, N, K)
    assert need > 0 and need % (M * N * 4) == 0 and 2 <= need // (M * N * 4) <= 8
    assert L.mslk_amd_debug_dispatch_name(M, N, K, 0, 0, 0, 1).decode().startswith("splitk_partial<64,64")
    assert "splitk" not in L.mslk_amd_debug_dispatch_name(M, N, K, 0, 0, 0, 0).decode()
    g = torch.Generator().manual_seed(M + N + K)
    xi, wi, xs, ws = _ints(M, K, g), _ints(N, K, g), _pow2(M, g), _pow2(N, g)
    bias = None if bias_dtype is None else torch.randint(-4, 5, (N,), generator=g).float()
    want = _want(xi, wi, xs, ws, bias, fp16_out)
    xq, wq, xsd, wsd = xi.to(F8).to(DEV), wi.to(F8).to(DEV), xs.to(DEV), ws.to(DEV)
    bd = None if bias is None else bias.to(bias_dtype).to(DEV)
    op = torch.ops.mslk.f8f8f16_rowwise if fp16_out else torch.ops.mslk.f8f8bf16_rowwise
    y = op(xq, wq, xsd, wsd, bias=bd)          # the operator passes the workspace
    torch.cuda.synchronize()
    _same_bits(y, want, f"split {M}x{N}x{K}")
    # without a workspace: the ordinary kernels, the same bits
    y2 = torch.full((M, N), SENTINEL, dtype=want.dtype, device=DEV)
    fn = L.mslk_amd_f8f8f16_rowwise if fp16_out else L.mslk_amd_f8f8bf16_rowwise
    _lib.check(fn(xq.data_ptr(), wq.data_ptr(), xsd.data_ptr(), wsd.data_ptr(), None if bd is None else bd.data_ptr(),
                  0 if bd is None else (1 if bias_dtype == torch.float32 else 2), y2.data_ptr(), M, N, K, None, 0,
                  torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    _same_bits(y2, want, f"unsplit {M}x{N}x{K}")


@pytest.mark.parametrize("fp16_out", [False, True])
@pytest.mark.parametrize("M,N,K", [(128, 512, 8192), (300, 528, 6208), (96, 2048, 16384)])
def test_k_split_on_preshuffled_weights_exact(M, N, K, fp16_out):
    """The K split reads blocked weights as well (a K slice of a 16-row group starts 16 x k0 bytes into the group); the
    operator passes the workspace, the entry point without one runs the unsplit kernels: the same bits from both."""
    from mslk_amd import _lib
    L = _lib.lib()
    assert L.mslk_amd_debug_dispatch_name(M, N, K, 0, 0, 1, 1).decode().startswith("splitk_partial<64,64,waves=4x1,ring=5> preshuffled")
    g = torch.Generator().manual_seed(M + N + K)
    xi, wi, xs, ws = _ints(M, K, g), _ints(N, K, g), _pow2(M, g), _pow2(N, g)
    bias = torch.randint(-4, 5, (N,), generator=g).float()
    want = _want(xi, wi, xs, ws, bias, fp16_out)
    xq, xsd, wsd, bd = xi.to(F8).to(DEV), xs.to(DEV), ws.to(DEV), bias.to(DEV)
    wshuf = mslk_amd.preshuffle_b_mfma(wi.to(F8).to(DEV))
    op = torch.ops.mslk.f8f8f16_rowwise_preshuffle if fp16_out else torch.ops.mslk.f8f8bf16_rowwise_preshuffle
    y = op(xq, wshuf, xsd, wsd, bias=bd)
    torch.cuda.synchronize()
    _same_bits(y, want, f"pre-shuffled, split {M}x{N}x{K}")
    y2 = torch.full((M, N), SENTINEL, dtype=want.dtype, device=DEV)
    _lib.check(L.mslk_amd_f8f8_rowwise_preshuffle(xq.data_ptr(), wshuf.data_ptr(), xsd.data_ptr(), wsd.data_ptr(), bd.data_ptr(), 1,
                                                  y2.data_ptr(), 1 if fp16_out else 0, M, N, K, torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    _same_bits(y2, want, f"pre-shuffled, unsplit {M}x{N}x{K}")


@pytest.mark.parametrize("M,N,K", [(1, 8192, 5248), (9, 1000, 5376), (16, 4096, 6784), (33, 2560, 5504), (48, 768, 11008), (64, 520, 11264),
                                   (4, 4096, 11008), (20, 1024, 2560)])
def test_weight_streaming_kernel_exact_on_k_loops_that_do_not_divide_among_its_waves(M, N, K):
    """M <= 64 on narrow weights: the weight-streaming kernel deals whole K steps of 128 bytes to its eight waves.  With
    K % 1024 != 0 (11008, 13824 and the like) the waves get unequal shares and the last batch is partly empty; the last
    two cases stay on the register-direct form of the kernel (few rows on few weight rows; a short K)."""
    from mslk_amd import _lib
    name = _lib.lib().mslk_amd_debug_dispatch_name(M, N, K, 2, 0, 0, 1).decode()
    assert name.startswith("skinny_registers" if (M, K) in ((4, 11008), (20, 2560)) else "skinny_lds"), name
    g = torch.Generator().manual_seed(M + N + K)
    xi, wi, xs, ws = _ints(M, K, g), _ints(N, K, g), _pow2(M, g), _pow2(N, g)
    bias = torch.randint(-4, 5, (N,), generator=g).float()
    y = torch.ops.mslk.f8f8bf16_rowwise(xi.to(F8).to(DEV), wi.to(F8).to(DEV), xs.to(DEV), ws.to(DEV), bias=bias.bfloat16().to(DEV))
    torch.cuda.synchronize()
    _same_bits(y, _want(xi, wi, xs, ws, bias), f"{M}x{N}x{K}")

