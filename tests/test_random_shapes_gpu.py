"""Seeded random shapes through the dense, stacked and TensorList operators with integer-valued codes and power-of-two
scales: fp32 accumulation is exact, so every output must match the fp32 product of the same numbers bit for bit.  The fixed
cases elsewhere pin each code path; this sweep walks combinations nobody wrote down (shape classes of the dispatch,
K loops of one to thirty-two steps with and without a tail, ragged groups next to empty ones).
Reference for the pattern: the case lists of test/gemm/gemm_test.py:169-219 (_fp8_gemm_cases) and 749-764 (grouped 2D-3D)."""
import random

import pytest
import torch

import mslk_amd  # noqa: F401  (registers the operators)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F8 = torch.float8_e4m3fn


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_shapes_are_bit_exact(seed):
    rnd = random.Random(seed)
    g = torch.Generator().manual_seed(rnd.randrange(1 << 30))
    ints = lambda r, k: torch.randint(-8, 9, (r, k), generator=g).float()
    pow2 = lambda n: 2.0 ** torch.randint(-3, 4, (n,), generator=g).float()
    for case in range(40):
        kind = rnd.choice(["dense", "dense", "dense_bias", "stacked", "tensorlist"])
        K = rnd.choice([128, 256, 272, 384, 512, 640, 1024, 2064, 4096])
        if kind.startswith("dense"):
            M = rnd.choice([1, 3, 16, 40, 64, 100, 256, 300, 1000, 2048, 2304, 3100, 4352])
            N = rnd.choice([256, 520, 1024, 2048, 4096, 5120, 8192])
            if M * N * K > 2 ** 34:
                K = 512
            xi, wi, xs, ws = ints(M, K), ints(N, K), pow2(M), pow2(N)
            want = (xi @ wi.T) * xs[:, None] * ws[None, :]
            bias = None
            if kind == "dense_bias":
                bias = torch.randint(-4, 5, (N,), generator=g).float()
                want = want + bias[None, :]
                bias = bias.to(rnd.choice([torch.float32, torch.bfloat16])).to(DEV)
            y = torch.ops.mslk.f8f8bf16_rowwise(xi.to(F8).to(DEV), wi.to(F8).to(DEV), xs.to(DEV), ws.to(DEV), bias=bias)
            assert torch.equal(y.cpu(), want.bfloat16()), f"seed {seed} case {case}: {kind} M={M} N={N} K={K}"
            continue
        G = rnd.choice([1, 3, 8, 16, 40])
        N = rnd.choice([512, 768, 1024, 2048])
        K = max(K, 512)   # the grouped operators refuse smaller K, as the reference does
        ms = [rnd.choice([0, 1, 17, 64, 65, 128, 200, 256, 300, 513, 1100]) for _ in range(G)]
        if sum(ms) == 0:
            ms[0] = 5
        xi, wi = [ints(m, K) for m in ms], [ints(N, K) for _ in ms]
        xs, ws = [pow2(m) for m in ms], [pow2(N) for _ in ms]
        want = [(a @ b.T) * c[:, None] * d[None, :] for a, b, c, d in zip(xi, wi, xs, ws)]
        where = f"seed {seed} case {case}: {kind} N={N} K={K} rows={ms}"
        if kind == "tensorlist":
            ys = torch.ops.mslk.f8f8bf16_rowwise_grouped([t.to(F8).to(DEV) for t in xi], [t.to(F8).to(DEV) for t in wi],
                                                         [t.to(DEV) for t in xs], [t.to(DEV) for t in ws])
            for e, (y, w) in enumerate(zip(ys, want)):
                assert torch.equal(y.cpu(), w.bfloat16()), f"{where}, group {e}"
        else:
            y = torch.ops.mslk.f8f8bf16_rowwise_grouped_stacked(torch.cat(xi).to(F8).to(DEV), torch.stack(wi).to(F8).to(DEV),
                                                                torch.cat(xs).to(DEV), torch.stack(ws).to(DEV),
                                                                torch.tensor(ms, dtype=torch.int64, device=DEV))
            assert torch.equal(y.cpu(), torch.cat(want).bfloat16()), where
