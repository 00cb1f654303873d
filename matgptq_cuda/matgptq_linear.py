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
        n_out, n_in = qweight.shape
        self.n_out_features, self.n_in_features = int(n_out), int(n_in)
        self.bitwidth, self.group_size = bitwidth, group_size
        # the storage type of the scales decides the arithmetic type of the layer (flag bit 1)
        flag = MatGTPQ_FeatureFlags.ASYNC
        if scales.dtype == torch.bfloat16:
            flag = flag | MatGTPQ_FeatureFlags.IS_BF16
        self.flag: int = int(flag)

        ops = torch.ops.matgptq_cuda
        shape = (self.n_out_features, self.n_in_features)

        def frozen(t: torch.Tensor) -> torch.nn.Parameter:
            return torch.nn.Parameter(t, requires_grad=False)

        def per_group(t: torch.Tensor) -> torch.Tensor:  # scales and zeros share one device layout
            return ops.reorder_matgptq_scales(t, *shape, self.group_size)

        self.matgptq_qweight = frozen(ops.pack_matgptq_qweights(qweight, *shape, self.bitwidth, self.group_size, self.flag))
        self.matgptq_scales = frozen(per_group(scales))
        self.matgptq_zeros = None if zeros is None else frozen(per_group(zeros.to(scales.dtype).contiguous()))
        if perm is None:
            self.matgptq_perm = None
        else:
            if perm.numel() != self.n_in_features:
                raise ValueError("perm must have n_in_features elements")
            self.register_buffer("matgptq_perm",
                                 perm.to(device=self.matgptq_qweight.device, dtype=torch.int64).reshape(-1))

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

    @torch.no_grad()
    def forward_prologue(self, kind: int, a: torch.Tensor, added=None, norm_weight=None, residual_out=None,
                         eps: float = 1e-5) -> torch.Tensor:
        """Additive: `forward` on activations that the kernel forms while it stages them (the SiLU gate
        of a fused gate_up output, or residual add + RMS norm; `matgptq_amd.ops.matmul_matgptq_prologue`).
        Up to four rows, fp16, group size 128, no act-order permutation."""
        from matgptq_amd import ops

        if self.matgptq_perm is not None:
            raise RuntimeError("the fused prologues do not apply to a layer with an act-order permutation")
        return ops.matmul_matgptq_prologue(kind, a, self.matgptq_qweight, self.matgptq_scales, self.matgptq_zeros,
                                           self.n_out_features, self.n_in_features, self.bitwidth, self.group_size,
                                           added, norm_weight, residual_out, eps)
