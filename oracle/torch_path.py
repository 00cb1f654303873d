"""The reference's CPU PyTorch path, restated with torch ops: slice -> dequantize -> F.linear
(src/quant_utils_matgpqt.py:9-22,202-224).  TEST / BASELINE INFRASTRUCTURE ONLY: bench.py's
`cpu_baseline` leg times it on the host cores; nothing shipped imports it.

It is pinned by tests/test_oracle_torch_path.py against the NumPy oracle and the golden
vectors (same integer formula, same two fp16 roundings, F.linear of torch itself).
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


def matryoshka_slice(x: torch.Tensor, master_bitwidth: int, slice_bitwidth: int) -> torch.Tensor:
    drop = 8 - slice_bitwidth  # always an 8-bit store (:10)
    floor = x >> drop
    if master_bitwidth == slice_bitwidth:
        return torch.clamp(floor, 0, 2 ** slice_bitwidth - 1)
    round_bit = (x >> (drop - 1)) & 1
    return torch.clamp(floor + round_bit, 0, 2 ** slice_bitwidth - 1)


def dequantize(q, scale, zero, master_bitwidth: int, slice_bitwidth: int) -> torch.Tensor:
    q_shifted = matryoshka_slice(q, master_bitwidth, slice_bitwidth) << (master_bitwidth - slice_bitwidth)
    return scale * (q_shifted - zero)


def get_weight(qweight, scale, zero, master_bitwidth: int, slice_bitwidth: int) -> torch.Tensor:
    n = qweight.shape[0]
    s = scale.view(n, -1, 1)
    z = zero.view(n, -1, 1)
    groups = s.shape[1]
    return dequantize(qweight.view(n, groups, -1), s, z, master_bitwidth, slice_bitwidth).view_as(qweight)


def forward(x, qweight, scale, zero, master_bitwidth: int, slice_bitwidth: int) -> torch.Tensor:
    """FakeMatryoshkaLinear.forward without perm and bias (:218-224)."""
    return F.linear(x, get_weight(qweight, scale, zero, master_bitwidth, slice_bitwidth))
