"""Seeded synthetic inputs for the five benchmark / parity configurations.

Everything is generated on the CPU with `torch.Generator().manual_seed(1000 + config)` so that a CPU
checker and the GPU see identical bits; callers move the tensors to the GPU themselves.
  cfg0  M=N=K=1024, x ~ N(0,1), w ~ N(0,0.02), no bias
  cfg1  M=N=K=4096, 1 % of x's K channels scaled x20
  cfg2  M=8192, N=28672, K=4096, outlier channels as cfg1, bf16 bias ~ N(0,0.01)
  cfg3  N=K=8192, M in {1,4,16,64}
  cfg4  16 experts, 8192 routed tokens split by a seeded multinomial over Zipf(1.1) popularity,
        N=8192, K=5120 per expert
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional

import torch


def _gen(cfg: int) -> torch.Generator:
    return torch.Generator().manual_seed(1000 + cfg)


def _randn_bf16(shape, gen, std: float = 1.0, chunk_rows: int = 4096) -> torch.Tensor:
    """randn * std -> bf16, produced in row chunks to bound the fp32 temporary."""
    rows = shape[0]
    out = torch.empty(shape, dtype=torch.bfloat16)
    for r0 in range(0, rows, chunk_rows):
        r1 = min(rows, r0 + chunk_rows)
        t = torch.randn((r1 - r0,) + tuple(shape[1:]), generator=gen)
        if std != 1.0:
            t *= std
        out[r0:r1] = t.to(torch.bfloat16)
    return out


def _activations(M: int, K: int, gen, outliers: bool) -> torch.Tensor:
    x = torch.randn(M, K, generator=gen)
    if outliers:
        idx = torch.randperm(K, generator=gen)[: K // 100]
        x[:, idx] *= 20
    return x.to(torch.bfloat16)


@dataclass
class DenseWorkload:
    name: str
    x: torch.Tensor                      # [M, K] bf16
    w: torch.Tensor                      # [N, K] bf16
    bias: Optional[torch.Tensor] = None  # [N] bf16


@dataclass
class GroupedWorkload:
    name: str
    counts: List[int]
    x: torch.Tensor                      # [sum(counts), K] bf16
    w: List[torch.Tensor] = field(default_factory=list)  # G x [N, K] bf16


def cfg0(M: int = 1024, N: int = 1024, K: int = 1024) -> DenseWorkload:
    g = _gen(0)
    return DenseWorkload("cfg0", _activations(M, K, g, False), _randn_bf16((N, K), g, 0.02))


def cfg1(M: int = 4096, N: int = 4096, K: int = 4096) -> DenseWorkload:
    g = _gen(1)
    return DenseWorkload("cfg1", _activations(M, K, g, True), _randn_bf16((N, K), g, 0.02))


def cfg2(M: int = 8192, N: int = 28672, K: int = 4096) -> DenseWorkload:
    g = _gen(2)
    x = _activations(M, K, g, True)
    w = _randn_bf16((N, K), g, 0.02)
    bias = (torch.randn(N, generator=g) * 0.01).to(torch.bfloat16)
    return DenseWorkload("cfg2", x, w, bias)


def cfg3_weight(N: int = 8192, K: int = 8192) -> torch.Tensor:
    return _randn_bf16((N, K), _gen(3), 0.02)


def cfg3_activations(M: int, K: int = 8192) -> torch.Tensor:
    g = torch.Generator().manual_seed(1003 * 100 + M)
    return _activations(M, K, g, False)


def cfg4_counts(experts: int = 16, tokens: int = 8192, gen: Optional[torch.Generator] = None) -> List[int]:
    g = gen if gen is not None else _gen(4)
    p = (torch.arange(experts, dtype=torch.float64) + 1.0) ** -1.1
    draws = torch.multinomial(p / p.sum(), tokens, replacement=True, generator=g)
    return torch.bincount(draws, minlength=experts).tolist()


def cfg4(experts: int = 16, tokens: int = 8192, N: int = 8192, K: int = 5120) -> GroupedWorkload:
    g = _gen(4)
    counts = cfg4_counts(experts, tokens, g)
    x = _activations(tokens, K, g, False)
    w = [_randn_bf16((N, K), g, 0.02) for _ in range(experts)]
    return GroupedWorkload("cfg4", counts, x, w)
