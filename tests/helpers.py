"""Shared helpers of the parity tests (the oracle is the checker, mslk_amd the thing checked)."""
import torch

from oracle import fp8_rowwise_oracle as O


def codes(t: torch.Tensor) -> torch.Tensor:
    """e4m3fn tensor -> uint8 codes on the CPU."""
    return t.detach().cpu().view(torch.uint8)


def bits32(t: torch.Tensor) -> torch.Tensor:
    return t.detach().cpu().contiguous().view(torch.int32)


def assert_quant_bit_exact(a_cpu: torch.Tensor, xq_gpu: torch.Tensor, scale_gpu: torch.Tensor, scale_ub=None, K_out=None):
    """GPU codes and scales must equal the oracle's, bit for bit.  NaN rows: the sign of a NaN
    product is unspecified, so NaN codes are compared modulo the sign bit."""
    ref_q, ref_s = O.quantize_fp8_row(a_cpu, scale_ub)
    K = a_cpu.shape[-1]
    got = codes(xq_gpu)
    if K_out is not None and K_out != K:
        assert got.shape[-1] == K_out
        assert (got[..., K:] == 0).all(), "padding columns must be zero"
        got = got[..., :K]
    want = codes(ref_q)
    nan_rows = torch.isnan(ref_s)
    if nan_rows.any():
        m = nan_rows[..., None].expand_as(want)
        assert ((got & 0x7F)[m] == (want & 0x7F)[m]).all()
        assert torch.equal(got[~m], want[~m])
        gs = scale_gpu.detach().cpu()
        assert torch.isnan(gs[nan_rows]).all()
        assert torch.equal(bits32(gs[~nan_rows]), bits32(ref_s[~nan_rows]))
    else:
        bad = (got != want)
        assert not bad.any(), f"{bad.sum().item()} of {bad.numel()} codes differ"
        assert torch.equal(bits32(scale_gpu), bits32(ref_s)), "scale bits differ"
    assert scale_gpu.shape == a_cpu.shape[:-1]


def assert_gemm_close(y_gpu: torch.Tensor, ref: torch.Tensor, what: str = "", rms: float = None):
    """north_star tolerance: max|y-ref|/max|ref| <= 1e-2 and ||y-ref||_F/||ref||_F <= 2e-3, plus the elementwise form the
    reference's own tests use (test/gemm/gemm_test.py:493-505): |y-ref| <= 1e-2 |ref| + 1e-2 rms(ref) for EVERY element,
    which a wrong small output element cannot hide behind a large one.

    One correct bf16 rounding alone costs up to 2^-8 relative per element (about 1.1e-3 normwise on
    average), so for outputs of fewer than 4096 elements -- where the norm does not average it out --
    the comparison is made against the oracle rounded to bf16 once.
    """
    if ref.numel() < 4096:
        ref = ref.to(torch.bfloat16).to(ref.dtype)
    max_rel, normwise = O.gemm_errors(y_gpu.float(), ref)
    assert max_rel <= O.MAX_REL_TOL, f"{what}: max-rel {max_rel:.3e} > {O.MAX_REL_TOL}"
    assert normwise <= O.NORMWISE_TOL, f"{what}: normwise {normwise:.3e} > {O.NORMWISE_TOL}"
    bad, worst = O.gemm_elementwise_violations(y_gpu.float(), ref, rms)
    assert bad == 0, f"{what}: {bad} elements beyond rtol {O.ELEM_RTOL} / atol {O.ELEM_ATOL_RMS} rms (worst {worst:.2f} x the bound)"
    return max_rel, normwise
