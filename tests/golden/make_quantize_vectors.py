"""Writes tests/golden/quantize_rows.json: hand-picked rows and the codes / scale bits that plain
CPU torch (the library the reference's torch branch is written in) produces for the formula of
mslk/quantize/triton/fp8_quantize.py:360-378.  The reference itself is not imported.

    python tests/golden/make_quantize_vectors.py
"""
import json
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import fp8_rowwise_oracle as O  # noqa: E402


def main():
    g = torch.Generator().manual_seed(20251125)
    K = 48
    rows = {
        "zeros": torch.zeros(K),
        "one_hot_negative": torch.zeros(K).index_fill_(0, torch.tensor([17]), -2.71875),
        "powers_of_two": 2.0 ** torch.arange(-24, 24).float(),
        "ties_at_448": torch.tensor([448.0, -448.0, 224.0, 1.0, 0.0009765625] + [0.0] * (K - 5)),
        "amax_3": torch.cat([torch.tensor([3.0, -3.0]), torch.linspace(-3, 3, K - 2)]),
        "subnormal_inputs": torch.full((K,), 1e-39),
        "bf16_max": torch.cat([torch.tensor([3.3895313892515355e38]), torch.randn(K - 1, generator=g) * 1e30]),
        "normal": torch.randn(K, generator=g),
        "outlier": torch.randn(K, generator=g).index_fill_(0, torch.tensor([3]), 950.0),
        "negative_zero": torch.tensor([-0.0, 0.0, 1.5, -1.5] + [0.25] * (K - 4)),
        "nan_row": torch.randn(K, generator=g).index_fill_(0, torch.tensor([9]), float("nan")),
    }
    cases = []
    for name, r in rows.items():
        for ub in (None, 1.25):
            a = r.to(torch.bfloat16).reshape(1, K)
            q, s = O.quantize_fp8_row(a, None if ub is None else torch.tensor([ub]))
            cases.append({
                "name": f"{name}{'' if ub is None else '_ub'}",
                "scale_ub": ub,
                "input_bf16_bits": (a.view(torch.int16).to(torch.int32) & 0xFFFF).tolist(),
                "codes": q.view(torch.uint8).tolist(),
                "scale_bits": s.view(torch.int32).tolist(),
            })
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "quantize_rows.json")
    with open(out, "w") as f:
        json.dump({"torch": torch.__version__, "cases": cases}, f)
    print(out, len(cases), "cases")


if __name__ == "__main__":
    main()
