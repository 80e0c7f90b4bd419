"""Pins the oracle (CPU only): the scalar C twin and the torch restatement must agree bit for bit,
and both must satisfy what the mathematics of the format fixes independently of either."""
import json
import os

import pytest
import torch

from oracle import c_twin
from oracle import fp8_rowwise_oracle as O

ALL_BF16 = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "quantize_rows.json")


def test_c_cast_matches_torch_on_all_bf16_and_random_fp32():
    f = ALL_BF16.float()
    t = f.to(torch.float8_e4m3fn).view(torch.uint8)
    c = c_twin.e4m3fn_cast(f)
    nan = torch.isnan(f)
    assert torch.equal(t[~nan], c[~nan])
    assert ((t[nan] & 0x7F) == 0x7F).all() and ((c[nan] & 0x7F) == 0x7F).all()
    g = torch.Generator().manual_seed(7)
    x = torch.randint(-2**31, 2**31 - 1, (4_000_000,), generator=g, dtype=torch.int64).to(torch.int32).view(torch.float32)
    nan = torch.isnan(x)
    assert torch.equal(x.to(torch.float8_e4m3fn).view(torch.uint8)[~nan], c_twin.e4m3fn_cast(x)[~nan])
    y = torch.rand(4_000_000, generator=g) * 1000 - 500  # dense around the representable range and the NaN edge
    assert torch.equal(y.to(torch.float8_e4m3fn).view(torch.uint8), c_twin.e4m3fn_cast(y))


def test_cast_known_answers():
    # OCP FP8 E4M3: bias 7, 3 mantissa bits, max 448 = 0x7E, subnormal step 2^-9, S.1111.111 = NaN.
    kat = [(0.0, 0x00), (-0.0, 0x80), (1.0, 0x38), (-1.0, 0xB8), (448.0, 0x7E), (-448.0, 0xFE), (2.0**-9, 0x01),
           (2.0**-10, 0x00), (3 * 2.0**-10, 0x02), (2.0**-6, 0x08), (1.0625, 0x38), (1.1875, 0x3A), (0.875, 0x36),
           (447.9, 0x7E), (463.9, 0x7E), (464.0, 0x7E), (464.1, 0x7F), (480.0, 0x7F), (1e9, 0x7F),
           (float("inf"), 0x7F), (240.0, 0x77), (256.0, 0x78), (17.0, 0x58), (19.0, 0x5A)]
    vals = torch.tensor([k for k, _ in kat], dtype=torch.float32)
    want = torch.tensor([v for _, v in kat], dtype=torch.uint8)
    assert torch.equal(c_twin.e4m3fn_cast(vals), want)
    assert torch.equal(vals.to(torch.float8_e4m3fn).view(torch.uint8), want)


def test_cast_decode_round_trip_all_codes():
    L = c_twin.lib()
    for code in range(256):
        v = L.oracle_e4m3fn_to_f32(code)
        if code & 0x7F == 0x7F:
            assert v != v
            continue
        assert L.oracle_e4m3fn_from_f32(v) == code
        assert torch.tensor([code], dtype=torch.uint8).view(torch.float8_e4m3fn).float().item() == v


def _rows_for_amax(amax_bits_list):
    """One row per amax: every finite bf16 value with |v| <= amax (zero-padded to a common length)."""
    fin = ALL_BF16[torch.isfinite(ALL_BF16.float())]
    rows = []
    for b in amax_bits_list:
        amax = torch.tensor([b], dtype=torch.int16).view(torch.bfloat16).float().item()
        rows.append(fin[fin.float().abs() <= amax])
    K = max(r.numel() for r in rows)
    out = torch.zeros(len(rows), K, dtype=torch.bfloat16)
    for i, r in enumerate(rows):
        out[i, : r.numel()] = r
    return out


def test_quantize_c_twin_equals_torch_exhaustive_bf16():
    # every bf16 amax in [2^-3, 2^3): 6 binades x 128 mantissas, each against every bf16 value below it
    amax_bits = list(range(0x3E00, 0x4100))
    for i in range(0, len(amax_bits), 96):
        a = _rows_for_amax(amax_bits[i : i + 96])
        q, s = O.quantize_fp8_row(a)
        cq, cs = c_twin.quantize_rows(a)
        assert torch.equal(q.view(torch.uint8), cq)
        assert torch.equal(s.view(torch.int32), cs.view(torch.int32))


def test_quantize_scales_all_positive_bf16_amax():
    # one-element rows: every positive finite bf16 as the row maximum (incl. subnormals and bf16 max)
    a = ALL_BF16[1:0x7F80].reshape(-1, 1).contiguous()
    q, s = O.quantize_fp8_row(a)
    cq, cs = c_twin.quantize_rows(a)
    assert torch.equal(s.view(torch.int32), cs.view(torch.int32))
    assert torch.equal(q.view(torch.uint8), cq)
    # the element equal to the row maximum always lands on +448 once amax >= eps
    big = a.float().reshape(-1) >= 1.01e-12
    assert (q.view(torch.uint8).reshape(-1)[big] == 0x7E).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_quantize_c_twin_equals_torch_random(dtype):
    g = torch.Generator().manual_seed(11)
    for rows, K, std in [(64, 4096, 1.0), (33, 777, 30.0), (128, 1, 1.0), (1, 128, 1e-3), (7, 9000, 1.0)]:
        a = (torch.randn(rows, K, generator=g) * std).to(dtype)
        a[0] = 0
        q, s = O.quantize_fp8_row(a)
        cq, cs = c_twin.quantize_rows(a)
        assert torch.equal(q.view(torch.uint8), cq)
        assert torch.equal(s.view(torch.int32), cs.view(torch.int32))
        ub = 0.75 * std
        q, s = O.quantize_fp8_row(a, torch.tensor([ub]))
        cq, cs = c_twin.quantize_rows(a, ub)
        assert torch.equal(q.view(torch.uint8), cq)
        assert torch.equal(s.view(torch.int32), cs.view(torch.int32))


def test_quantize_closed_forms():
    # amax = 448 * 2^k: inv = 2^-k and scale = 2^k exactly; codes are the plain e4m3 rounding of a * 2^-k
    for k in (-4, 0, 3):
        amax = 448.0 * 2.0**k
        a = torch.tensor([[amax, -amax / 2, amax / 448, 0.0, -0.0, 3 * amax / 7]], dtype=torch.bfloat16)
        for q, s in (O.quantize_fp8_row(a), c_twin.quantize_rows(a)):
            assert s.item() == 2.0**k
            want = (a.float() * 2.0**-k).to(torch.float8_e4m3fn).view(torch.uint8)
            assert torch.equal(q.view(torch.uint8), want)
            assert q.view(torch.uint8)[0, 4].item() == 0x80  # -0.0 keeps its sign
    # zero row: amax clamps to bf16(1e-12) = 0x2B8D; all codes 0; scale = 1/(fl(1/eps)*448)
    z = torch.zeros(1, 64, dtype=torch.bfloat16)
    eps = torch.tensor([0x2B8D], dtype=torch.int16).view(torch.bfloat16).float()
    assert eps.item() == 1.0018652574217413e-12
    inv = (1.0 / eps) * 448.0
    for q, s in (O.quantize_fp8_row(z), c_twin.quantize_rows(z)):
        assert (q.view(torch.uint8) == 0).all()
        assert s.item() == (1.0 / inv).item() == 2.236306529429413e-15
    # fp16 input: 1e-12 is 0 in fp16, a zero row hits the inf -> 1.0 rule
    zh = torch.zeros(1, 8, dtype=torch.float16)
    for q, s in (O.quantize_fp8_row(zh), c_twin.quantize_rows(zh)):
        assert s.item() == 1.0 and (q.view(torch.uint8) == 0).all()
    # one-hot row: the single non-zero becomes +-448, everything else 0
    oh = torch.zeros(1, 100, dtype=torch.bfloat16)
    oh[0, 37] = -3.140625
    for q, s in (O.quantize_fp8_row(oh), c_twin.quantize_rows(oh)):
        c = q.view(torch.uint8)
        assert c[0, 37].item() == 0xFE and c.sum().item() == 0xFE
    # NaN anywhere in the row poisons the whole row
    n = torch.ones(1, 16, dtype=torch.bfloat16)
    n[0, 5] = float("nan")
    for q, s in (O.quantize_fp8_row(n), c_twin.quantize_rows(n)):
        assert torch.isnan(s).all() and ((q.view(torch.uint8) & 0x7F) == 0x7F).all()


def test_quantize_invariants():
    g = torch.Generator().manual_seed(3)
    a = (torch.randn(256, 1024, generator=g) * torch.logspace(-6, 6, 256)[:, None]).to(torch.bfloat16)
    q, s = O.quantize_fp8_row(a)
    assert (s > 0).all()
    c = q.view(torch.uint8)
    assert ((c & 0x7F) == 0x7E).any(dim=1).all(), "every non-zero row holds a +-448 code"
    assert ((c & 0x7F) != 0x7F).all(), "no NaN codes without scale_ub"
    deq = q.float() * s[:, None]
    err = (deq - a.float()).abs()
    # half an e4m3 ulp of the scaled value, plus the rounding of inv and scale (2 ulp of fp32 each)
    half_ulp = torch.maximum(deq.abs() * 2.0**-4, s[:, None] * 2.0**-10)
    assert (err <= half_ulp * (1 + 1e-5) + a.float().abs() * 4e-7).all()
    # codes are monotone in the input within a row
    order = a.float().argsort(dim=1)
    qs = torch.gather(q.float(), 1, order)
    assert (qs[:, 1:] >= qs[:, :-1]).all()


def test_dequant_matmul_against_brute_force_and_identities():
    g = torch.Generator().manual_seed(5)
    M, N, K = 7, 9, 37
    xq = torch.randint(0, 256, (M, K), generator=g, dtype=torch.int64).to(torch.uint8)
    wq = torch.randint(0, 256, (N, K), generator=g, dtype=torch.int64).to(torch.uint8)
    xq[(xq & 0x7F) == 0x7F] = 0x10
    wq[(wq & 0x7F) == 0x7F] = 0x10
    xs = torch.rand(M, generator=g) + 0.5
    ws = torch.rand(N, generator=g) * 0.01
    bias = torch.randn(N, generator=g)
    brute = c_twin.dequant_gemm(xq, wq, xs, ws, bias)
    got = O.dequant_matmul(xq.view(torch.float8_e4m3fn), wq.view(torch.float8_e4m3fn), xs, ws, bias, dtype=torch.float64)
    assert torch.allclose(got, brute, rtol=1e-12, atol=1e-12)
    got32 = O.dequant_matmul(xq.view(torch.float8_e4m3fn), wq.view(torch.float8_e4m3fn), xs, ws, bias)
    assert torch.allclose(got32.double(), brute, rtol=1e-4, atol=1e-4)
    # identity weights select the dequantized activations
    K = 16
    eye = torch.eye(K).to(torch.float8_e4m3fn)
    x = torch.randn(5, K, generator=g).bfloat16()
    q, s = O.quantize_fp8_row(x)
    y = O.dequant_matmul(q, eye, s, torch.ones(K))
    assert torch.equal(y, O.dequantize_fp8_row(q, s))
    # the reference's CPU fallback (bf16 matmul, scaled afterwards) agrees within bf16 rounding
    x = torch.randn(64, 256, generator=g).bfloat16()
    w = (torch.randn(48, 256, generator=g) * 0.02).bfloat16()
    xq_, xs_ = O.quantize_fp8_row(x)
    wq_, ws_ = O.quantize_fp8_row(w)
    ref = O.dequant_matmul(xq_, wq_, xs_, ws_)
    cpu = O.matmul_fp8_row_cpu(xq_, wq_, xs_, ws_)
    max_rel, normwise = O.gemm_errors(cpu.float(), ref)
    assert max_rel < 2e-2 and normwise < 8e-3


def test_golden_quantize_rows():
    """Vectors committed under tests/golden (made by tests/golden/make_quantize_vectors.py with plain
    torch): guards the oracle against drift of the library routines it is written in."""
    with open(GOLDEN) as f:
        data = json.load(f)
    for case in data["cases"]:
        a = torch.tensor(case["input_bf16_bits"], dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
        ub = None if case["scale_ub"] is None else torch.tensor([case["scale_ub"]])
        q, s = O.quantize_fp8_row(a, ub)
        cq, cs = c_twin.quantize_rows(a, case["scale_ub"])
        want_q = torch.tensor(case["codes"], dtype=torch.uint8)
        want_s = torch.tensor(case["scale_bits"], dtype=torch.int32)
        nan = want_q.new_tensor([(b & 0x7F800000) == 0x7F800000 and (b & 0x7FFFFF) != 0 for b in case["scale_bits"]]).bool()
        for got_q, got_s in ((q.view(torch.uint8), s), (cq, cs)):
            assert torch.equal(got_q[~nan], want_q[~nan]), case["name"]
            assert torch.equal(got_s.view(torch.int32)[~nan], want_s[~nan]), case["name"]


def test_jagged_rows_are_zero_rows_and_live_rows_are_untouched():
    g = torch.Generator().manual_seed(77)
    a = torch.randn(3, 5, 7, 24, generator=g).bfloat16()
    zs = torch.randint(0, 8, (3, 5), generator=g)
    q, s = O.quantize_fp8_row_jagged(a, zs)
    q0, s0 = O.quantize_fp8_row(a)
    zero_row_scale = O.quantize_fp8_row(torch.zeros(1, 24, dtype=torch.bfloat16))[1].item()
    assert zero_row_scale == 2.236306529429413e-15   # 1 / fl32(fl32(1 / bf16(1e-12)) * 448)
    for b in range(3):
        for m in range(5):
            k = int(zs[b, m])
            assert torch.equal(q[b, m, :k].view(torch.uint8), q0[b, m, :k].view(torch.uint8))
            assert torch.equal(s[b, m, :k], s0[b, m, :k])
            assert (q[b, m, k:].view(torch.uint8) == 0).all()
            assert (s[b, m, k:] == zero_row_scale).all()
    # lower-rank inputs are grouped by their second-to-last dimension
    a2 = torch.randn(20, 30, generator=g).bfloat16()
    q, s = O.quantize_fp8_row_jagged(a2, torch.tensor([6]))
    assert (q[6:].view(torch.uint8) == 0).all() and torch.equal(s[:6], O.quantize_fp8_row(a2)[1][:6])


def test_dequantize_closed_forms():
    codes = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).reshape(1, 256)
    # scale 1: every finite e4m3fn value is exactly representable in bf16
    d = O.dequantize_fp8_row_bf16(codes, torch.ones(1))
    ref = codes.to(torch.float32)
    ok = ~torch.isnan(ref)
    assert torch.equal(d.float()[ok], ref[ok]) and torch.isnan(d.float()[~ok]).all()
    # powers of two scale exactly; 448 * 2^-10 etc. stay normal in bf16
    for e in (-10, -3, 4):
        d = O.dequantize_fp8_row_bf16(codes, torch.tensor([2.0 ** e]))
        assert torch.equal(d.float()[ok], ref[ok] * 2.0 ** e)
    # roundings worked by hand (bf16 spacing in [1, 2) is 2^-7):
    one = torch.tensor([[1.0]]).to(torch.float8_e4m3fn)
    assert O.dequantize_fp8_row_bf16(one, torch.tensor([1.0 + 2.0 ** -8])).item() == 1.0            # tie -> even
    assert O.dequantize_fp8_row_bf16(one, torch.tensor([1.0 + 3 * 2.0 ** -8])).item() == 1.015625   # tie -> even (up)
    x175 = torch.tensor([[1.75]]).to(torch.float8_e4m3fn)
    assert O.dequantize_fp8_row_bf16(x175, torch.tensor([1.0 + 2.0 ** -8])).item() == 1.7578125     # 1.7568359375 -> up
    x15 = torch.tensor([[1.5]]).to(torch.float8_e4m3fn)
    assert O.dequantize_fp8_row_bf16(x15, torch.tensor([1.0 + 2.0 ** -9])).item() == 1.5            # 1.5029296875 -> down
    # round trip: e4m3fn keeps 3 mantissa bits, bf16 7
    g = torch.Generator().manual_seed(3)
    a = torch.randn(64, 256, generator=g).bfloat16()
    q, sc = O.quantize_fp8_row(a)
    back = O.dequantize_fp8_row_bf16(q, sc).float()
    amax = a.float().abs().amax(dim=1, keepdim=True)
    assert ((back - a.float()).abs() <= a.float().abs() * 2.0 ** -4 + amax * 2.0 ** -9).all()


def test_saturating_quantization_closed_forms():
    # amax = 448 * 2^k: s = 2^-k exactly, scale = 2^k, every value v * 2^-k is converted exactly as is
    for k in (-3, 0, 5):
        y = torch.tensor([[448.0, -224.0, 1.0, 0.0, 17.0, -0.4375]]) * 2.0 ** k
        q, sc = O.quantize_rows_saturating(y)
        assert sc.item() == 2.0 ** k
        assert q.view(torch.uint8).tolist() == [[0x7E, 0xF6, 0x38, 0x00, 0x58, 0xAE]]   # 17 -> 16 (tie to even), -0.4375 exact
    # scale_ub below the maximum: larger values saturate at +-448 (0x7E / 0xFE) instead of becoming NaN
    y = torch.tensor([[100.0, -50.0, 25.0, 10.0]])
    q, sc = O.quantize_rows_saturating(y, torch.tensor([25.0]))
    assert sc.item() == torch.tensor(1.0) / (torch.tensor(448.0) / torch.tensor(25.0))
    assert q.view(torch.uint8)[0, :3].tolist() == [0x7E, 0xFE, 0x7E]
    assert q.float()[0, 3].item() == 176.0    # 10 * 17.92 = 179.2 -> grid {160, 176, 192}
    # zero row: the clamp at 1e-12 decides the scale
    q, sc = O.quantize_rows_saturating(torch.zeros(1, 8))
    assert (q.view(torch.uint8) == 0).all() and sc.item() == (torch.tensor(1.0) / (torch.tensor(448.0) / torch.tensor(1e-12))).item()
    # on rows where both formulas are exact they agree with the stand-alone quantizer
    g = torch.Generator().manual_seed(8)
    y = torch.randn(16, 64, generator=g)
    y[:, 0] = 448.0 * 2.0 ** torch.randint(-4, 4, (16,), generator=g).float()
    y = torch.minimum(y.abs(), y[:, :1]) * torch.sign(y)
    q1, s1 = O.quantize_rows_saturating(y)
    q2, s2 = O.quantize_fp8_row(y)
    assert torch.equal(q1.view(torch.uint8), q2.view(torch.uint8)) and torch.equal(s1, s2)


def test_fused_producers_reduce_to_their_parts():
    g = torch.Generator().manual_seed(9)
    x0 = torch.randn(5, 40, generator=g).bfloat16()
    x1 = torch.randn(5, 40, generator=g).bfloat16()
    q, sc = O.silu_mul_quant(x0, x1)
    # silu(0) = 0 and silu(x) -> x for large x: closed-form rows
    big = torch.full((1, 8), 30.0).bfloat16()
    q2, s2 = O.silu_mul_quant(big, torch.tensor([[1.0, 2.0, 4.0, -8.0, 0.5, 0.0, 1.0, 1.0]]).bfloat16())
    assert s2.item() == (torch.tensor(1.0) / (torch.tensor(448.0) / torch.tensor(240.0))).item()
    assert q2.float()[0].tolist() == [56.0, 112.0, 224.0, -448.0, 28.0, 0.0, 56.0, 56.0]
    qz, _ = O.silu_mul_quant(torch.zeros(1, 8).bfloat16(), big)
    assert (qz.view(torch.uint8) == 0).all()
    # independent evaluation in float64
    y64 = (x0.double() * torch.sigmoid(x0.double()) * x1.double())
    back = q.float() * sc[:, None]
    assert ((back - y64.float()).abs() <= y64.abs().float() * 2.0 ** -4 + y64.abs().amax(dim=1, keepdim=True).float() * 2.0 ** -9).all()
    # gather: a permutation with unit scores is a row permutation of the plain quantization
    x = torch.randn(7, 32, generator=g).bfloat16()
    perm = torch.randperm(7, generator=g)
    qg, sg = O.gather_scale_quant_dense_tokens(x, perm, torch.zeros(7, dtype=torch.int64), torch.ones(7, 1))
    qp, sp = O.quantize_rows_saturating(x.float())
    assert torch.equal(qg.view(torch.uint8), qp.view(torch.uint8)[perm]) and torch.equal(sg, sp[perm])
    # a power-of-two score only moves the scale
    sc2 = torch.full((7, 3), 1.0)
    sc2[:, 2] = 4.0
    qg2, sg2 = O.gather_scale_quant_dense_tokens(x, perm, torch.full((7,), 2), sc2)
    assert torch.equal(qg2.view(torch.uint8), qg.view(torch.uint8)) and torch.equal(sg2, sg * 4.0)


def test_preshuffle_layout_by_brute_force():
    """Element (n, k) must land at flat position ((n // 16) * (K // 64) + k // 64) * 1024 + ((k % 64) // 16) * 256 + (n % 16) * 16 + k % 16."""
    for lead, N, K in [((), 16, 64), ((), 48, 192), ((3,), 32, 128)]:
        count = N * K * (lead[0] if lead else 1)
        src = torch.arange(count, dtype=torch.int32).reshape(*lead, N, K)
        out = O.preshuffle_b(src)
        flat_src = src.reshape(-1, N, K)
        flat_out = out.reshape(-1, N * K)
        for gi in range(flat_src.shape[0]):
            for n in range(N):
                for k in range(0, K, 7):   # every 7th column keeps the loop short and still hits all residues
                    pos = ((n // 16) * (K // 64) + k // 64) * 1024 + ((k % 64) // 16) * 256 + (n % 16) * 16 + k % 16
                    assert flat_out[gi, pos] == flat_src[gi, n, k]
    # it is a permutation: sorting recovers the input
    assert torch.equal(out.reshape(-1).sort().values, src.reshape(-1))


def test_triton_arithmetic_closed_forms():
    # amax = 448 * 2^k: scale = 2^k and every x / 2^k is converted as is
    for k in (-3, 0, 5):
        y = (torch.tensor([[448.0, -224.0, 1.0, 0.0, 17.0, -0.4375]]) * 2.0 ** k).bfloat16()
        q, sc = O.quantize_fp8_row_triton_arithmetic(y)
        assert sc.item() == 2.0 ** k
        assert q.view(torch.uint8).tolist() == [[0x7E, 0xF6, 0x38, 0x00, 0x58, 0xAE]]
    # zero row: amax is raised to eps = 1/512 -> scale = 2^-9 / 448
    q, sc = O.quantize_fp8_row_triton_arithmetic(torch.zeros(1, 8).bfloat16())
    assert (q.view(torch.uint8) == 0).all() and sc.item() == (torch.tensor(2.0 ** -9) / torch.tensor(448.0)).item()
    # rows below eps are quantized against eps, not against their own maximum: 2^-12 / (2^-9 / 448) = 56
    q, sc = O.quantize_fp8_row_triton_arithmetic(torch.tensor([[2.0 ** -12, -2.0 ** -13]]).bfloat16())
    assert q.float().tolist() == [[56.0, -28.0]]
    # scale_ub below the maximum saturates (the torch branch produces NaN codes there)
    y = torch.tensor([[100.0, -50.0, 25.0, 10.0]]).bfloat16()
    q, sc = O.quantize_fp8_row_triton_arithmetic(y, torch.tensor([25.0]))
    assert sc.item() == (torch.tensor(25.0) / torch.tensor(448.0)).item()
    assert q.view(torch.uint8)[0, :3].tolist() == [0x7E, 0xFE, 0x7E] and q.float()[0, 3].item() == 176.0
    qt, _ = O.quantize_fp8_row(y, torch.tensor([25.0]))
    assert torch.isnan(qt.float()[0, 0])
    # the two arithmetics agree except in the last place of a few codes
    g = torch.Generator().manual_seed(10)
    a = torch.randn(64, 512, generator=g).bfloat16()
    q1, s1 = O.quantize_fp8_row_triton_arithmetic(a)
    q2, s2 = O.quantize_fp8_row(a)
    assert torch.allclose(s1, s2, rtol=3e-7, atol=0)
    diff = (q1.view(torch.uint8).int() - q2.view(torch.uint8).int()).abs()
    assert diff.max() <= 1 and (diff != 0).float().mean() < 1e-2


def test_elementwise_criterion_counts_what_it_should():
    ref = torch.tensor([[100.0, -100.0, 0.0, 1.0]], dtype=torch.float32)      # rms = sqrt(20001 / 4) = 70.71
    assert O.gemm_elementwise_violations(ref.clone(), ref) == (0, 0.0)
    y = ref.clone()
    y[0, 0] = 101.7                      # bound 1e-2 * 100 + 1e-2 * 70.71 = 1.707: just inside
    y[0, 2] = 0.70                       # bound 0.7071: inside
    assert O.gemm_elementwise_violations(y, ref)[0] == 0
    y[0, 1] = -101.8                     # beyond 1.707
    y[0, 3] = 1.8                        # |diff| 0.8 > 1e-2 + 0.7071
    bad, worst = O.gemm_elementwise_violations(y, ref)
    assert bad == 2 and abs(worst - 0.8 / (0.01 + 0.70712)) < 1e-3
    # a block of a larger tensor: the caller's rms replaces the block's own
    assert O.gemm_elementwise_violations(y, ref, rms=1000.0)[0] == 0



def test_reciprocal_fma_division_gives_the_codes_of_the_ieee_division():
    """The quantizer's Triton-arithmetic mode replaces x / s by r = 1 / s, q0 = x r, e = fma(-q0, s, x), q = e == 0 ? q0 :
    fma(e, r, q0) in rows whose maximum is a bf16 / fp16 value of at least 2^-64.  Exhaustive over every such maximum and every
    element not above it (2 x 10^9 pairs, split over threads): the e4m3 codes are the same.  Below 2^-64 the forms do differ
    (which is why the kernel divides there)."""
    from concurrent.futures import ThreadPoolExecutor
    jobs = []
    bf16_lo, bf16_hi = 0x1F80, 0x7F80                      # 2^-64 ... the first non-finite bf16
    edges = [bf16_lo, 0x4C00, 0x5E00, 0x6A00, 0x7300, 0x7A00, bf16_hi]   # the work per maximum grows with its bits
    for lo, hi in zip(edges[:-1], edges[1:]):
        jobs.append((torch.bfloat16, lo, hi))
    jobs += [(torch.float16, 1, 0x5000), (torch.float16, 0x5000, 0x6A00), (torch.float16, 0x6A00, 0x7C00)]
    with ThreadPoolExecutor(max_workers=8) as ex:
        results = list(ex.map(lambda j: c_twin.count_division_mismatches(*j), jobs))
    assert [r[0] for r in results] == [0] * len(jobs), results
    n, first, last = c_twin.count_division_mismatches(torch.bfloat16, 0x0400, 0x0C00)
    assert n > 0 and (last >> 16) < 0x1F80                 # tiny maxima: the two forms disagree somewhere
