"""`MatGPTQLinear` and `MatGTPQ_FeatureFlags` with the reference's interface
(inference_lib/matgptq_cuda/matgptq_linear.py:6-59)."""
from enum import IntEnum
from typing import Optional

import torch

import matgptq_cuda  # noqa: F401  (registers the operators)


class MatGTPQ_FeatureFlags(IntEnum):
    SYNC = 0
    ASYNC = 1
    IS_BF16 = 2


class MatGPTQLinear(torch.nn.Module):
    """Linear layer over packed b-bit codes.

    qweight : uint8 [N, K], codes already sliced to `bitwidth` (host or GPU tensor)
    scales  : [N, K / group_size] ([N, 1] for group_size -1), fp16
    zeros   : optional extension - per-group zero points in master-code units, same shape
              as `scales`; absent means 128 everywhere, the reference kernel's symmetric form
    perm    : optional extension - the quantiser's act-order column permutation [K]: the codes are
              stored in permuted column order and the input features are gathered with it before
              the product, `x[..., perm]`, as the reference's fake-quantised layer does
              (src/quant_utils_matgpqt.py:218-220); its kernel path has no counterpart
    forward returns a 2-D [batch, N] tensor without bias, like the reference.
    """

    def __init__(self, qweight: torch.Tensor, scales: torch.Tensor, bitwidth: int, group_size: int,
                 zeros: Optional[torch.Tensor] = None, perm: Optional[torch.Tensor] = None):
        super().__init__()
        self.n_out_features: int = qweight.shape[0]
        self.n_in_features: int = qweight.shape[1]
        self.bitwidth: int = bitwidth
        self.group_size: int = group_size

        self.flag: int = MatGTPQ_FeatureFlags.ASYNC + MatGTPQ_FeatureFlags.IS_BF16 * (scales.dtype == torch.bfloat16)

        self.matgptq_qweight = torch.nn.Parameter(
            torch.ops.matgptq_cuda.pack_matgptq_qweights(
                qweight, self.n_out_features, self.n_in_features, self.bitwidth, self.group_size, self.flag),
            requires_grad=False)
        self.matgptq_scales = torch.nn.Parameter(
            torch.ops.matgptq_cuda.reorder_matgptq_scales(
                scales, self.n_out_features, self.n_in_features, self.group_size),
            requires_grad=False)
        if zeros is not None:
            self.matgptq_zeros = torch.nn.Parameter(
                torch.ops.matgptq_cuda.reorder_matgptq_scales(
                    zeros.to(scales.dtype).contiguous(), self.n_out_features, self.n_in_features, self.group_size),
                requires_grad=False)
        else:
            self.matgptq_zeros = None
        if perm is not None:
            if perm.numel() != self.n_in_features:
                raise ValueError("perm must have n_in_features elements")
            self.register_buffer("matgptq_perm", perm.to(device=self.matgptq_qweight.device, dtype=torch.int64).reshape(-1))
        else:
            self.matgptq_perm = None

    @torch.no_grad()
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.matgptq_perm is not None:
            x = torch.index_select(x, -1, self.matgptq_perm)
        if self.matgptq_zeros is not None:
            return torch.ops.matgptq_cuda.matmul_matgptq_zp(
                x, self.matgptq_qweight, self.matgptq_scales, self.matgptq_zeros,
                self.n_out_features, self.n_in_features, self.bitwidth, self.group_size, self.flag)
        return torch.ops.matgptq_cuda.matmul_matgptq(
            x, self.matgptq_qweight, self.matgptq_scales,
            self.n_out_features, self.n_in_features, self.bitwidth, self.group_size, self.flag)
