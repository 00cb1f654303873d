"""Python face of the operators.

Reference operators (same names, argument meaning and errors as
inference_lib/matgptq_cuda/__init__.py:5-63):

    pack_matgptq_qweights(qweights, n_out_features, n_in_features, bitwidth, group_size, feature_flag)
    reorder_matgptq_scales(scales, n_out_features, n_in_features, group_size)
    matmul_matgptq(input, matgptq_weights, matgptq_scales, n_out_features, n_in_features,
                   bitwidth, group_size, feature_flag)

Additive operators of this implementation (all under torch.ops.matgptq_cuda):

    pack_matgptq_master      same signature as pack_matgptq_qweights, but takes 8-bit master
                             codes and slices them to `bitwidth` while packing
    matmul_matgptq_zp        matmul_matgptq with a per-group zero tensor (reordered with
                             reorder_matgptq_scales) after matgptq_scales
    unpack_matgptq_qweights  packed -> uint8 codes (tests, bit-exactness checks)
    slice_matgptq_master     rounded MSB slice of master codes on the GPU
    dequantize_matgptq       packed -> dense fp16 weight, rounded like the reference's dequantize
    pack_matgptq_master_resident    8-bit master codes [N, K] -> bit planes, most significant first
                                    (N*K/4 words): one buffer that serves every bitwidth
    matmul_matgptq_master           matmul_matgptq_zp on those planes with `bitwidth` as a run-time
                                    argument: the rounded slice is formed in registers
    unpack_matgptq_master_resident  planes -> the uint8 codes the GEMM sees at `bitwidth`

and, as a plain function over the C ABI (not a registered operator):

    matmul_matgptq_prologue  the decode product with the operator in front of it fused into the kernel
                             (SiLU gate of a fused gate_up output, or residual add + RMS norm)
"""
from __future__ import annotations

import torch

_ops = torch.ops.matgptq_cuda

pack_matgptq_qweights = _ops.pack_matgptq_qweights
pack_matgptq_master = _ops.pack_matgptq_master
reorder_matgptq_scales = _ops.reorder_matgptq_scales
matmul_matgptq = _ops.matmul_matgptq
matmul_matgptq_zp = _ops.matmul_matgptq_zp
unpack_matgptq_qweights = _ops.unpack_matgptq_qweights
slice_matgptq_master = _ops.slice_matgptq_master
dequantize_matgptq = _ops.dequantize_matgptq
pack_matgptq_master_resident = _ops.pack_matgptq_master_resident
unpack_matgptq_master_resident = _ops.unpack_matgptq_master_resident
matmul_matgptq_master = _ops.matmul_matgptq_master


def _out_dtype(feature_flag: int) -> torch.dtype:
    return torch.bfloat16 if feature_flag & 2 else torch.float16


# Shape rule of the reference's fake implementation (__init__.py:49-63), with leading
# dimensions folded into the batch like the kernel wrapper does.
@torch.library.register_fake("matgptq_cuda::matmul_matgptq")
def _matmul_fake(input, matgptq_weights, matgptq_scales, n_out_features, n_in_features,
                 bitwidth, group_size, feature_flag):
    m = input.numel() // n_in_features
    return input.new_empty((m, n_out_features), dtype=_out_dtype(feature_flag))


@torch.library.register_fake("matgptq_cuda::matmul_matgptq_zp")
def _matmul_zp_fake(input, matgptq_weights, matgptq_scales, matgptq_zeros, n_out_features,
                    n_in_features, bitwidth, group_size, feature_flag):
    m = input.numel() // n_in_features
    return input.new_empty((m, n_out_features), dtype=_out_dtype(feature_flag))


@torch.library.register_fake("matgptq_cuda::matmul_matgptq_master")
def _matmul_master_fake(input, planes, matgptq_scales, matgptq_zeros, n_out_features, n_in_features,
                        bitwidth, group_size, feature_flag):
    m = input.numel() // n_in_features
    return input.new_empty((m, n_out_features), dtype=_out_dtype(feature_flag))


@torch.library.register_fake("matgptq_cuda::dequantize_matgptq")
def _dequant_fake(matgptq_weights, matgptq_scales, matgptq_zeros, n_out_features, n_in_features,
                  bitwidth, group_size):
    return matgptq_scales.new_empty((n_out_features, n_in_features))


@torch.library.register_fake("matgptq_cuda::slice_matgptq_master")
def _slice_fake(master, bitwidth):
    return torch.empty_like(master)


def matryoshka_slice(x: torch.Tensor, master_bitwidth: int, slice_bitwidth: int) -> torch.Tensor:
    """Rounded MSB slice of uint8 master codes: the function the reference's callers apply
    before packing (src/quant_utils_matgpqt.py:9-17; used at inference_lib/vllm_matgptq.py:154
    and inference_lib/inference_demo_transformers.py:31).  GPU tensors of the 8-bit master
    take the HIP kernel; anything else is computed with the same integer formula in torch.
    """
    if x.dtype != torch.uint8:
        raise TypeError("master codes must be uint8")
    if master_bitwidth == slice_bitwidth and slice_bitwidth == 8:
        return x.clone()
    if x.is_cuda and master_bitwidth == 8 and slice_bitwidth in (2, 3, 4, 6):
        return slice_matgptq_master(x.contiguous(), slice_bitwidth)
    drop = 8 - slice_bitwidth  # the store is always 8 bits wide
    v = x.to(torch.int16)
    floor = v >> drop
    top = (1 << slice_bitwidth) - 1
    if master_bitwidth == slice_bitwidth:
        return floor.clamp_(0, top).to(torch.uint8)
    return (floor + ((v >> (drop - 1)) & 1)).clamp_(0, top).to(torch.uint8)


PRE_SILU_MUL, PRE_ADD_RMSNORM = 1, 2


def prologue_applies(kind: int, rows: int, n_in_features: int, group_size: int, dtype: torch.dtype) -> bool:
    """Whether `matmul_matgptq_prologue` covers this call (include/matgptq_abi.h: fp16 storage,
    group size 128, up to four rows; the norm needs all of K inside one round: K <= 8192)."""
    return (dtype == torch.float16 and group_size == 128 and 1 <= rows <= 4 and n_in_features % 128 == 0
            and (kind == PRE_SILU_MUL or (kind == PRE_ADD_RMSNORM and n_in_features <= 8192)))


def matmul_matgptq_prologue(kind: int, a: torch.Tensor, matgptq_weights: torch.Tensor, matgptq_scales: torch.Tensor,
                            matgptq_zeros, n_out_features: int, n_in_features: int, bitwidth: int, group_size: int,
                            added=None, norm_weight=None, residual_out=None, eps: float = 1e-5) -> torch.Tensor:
    """`matmul_matgptq[_zp]` on activations the kernel forms itself while staging them:

    PRE_SILU_MUL     a [M, 2K] = (gate | up)  ->  x = silu(gate) * up
    PRE_ADD_RMSNORM  a [M, K] the residual stream; v = a + added (added may be None), x = rms_norm(v) *
                     norm_weight; v is written to `residual_out` (not a or `added`) when given

    Launches on the current stream, allocates only the output; raises where the fused kernel does not
    apply (see `prologue_applies`)."""
    from . import _lib

    rows = a.shape[0]
    for t in (a, added, norm_weight, residual_out):
        if t is not None and (t.dtype != torch.float16 or not t.is_cuda or not t.is_contiguous()):
            raise ValueError("matmul_matgptq_prologue: contiguous float16 tensors on the GPU expected")
    width = 2 * n_in_features if kind == PRE_SILU_MUL else n_in_features
    if a.dim() != 2 or a.shape[1] != width:
        raise ValueError("matmul_matgptq_prologue: input has the wrong shape")
    for t in (added, residual_out):
        if t is not None and t.shape != a.shape:
            raise ValueError("matmul_matgptq_prologue: added tensor and residual output take the input's shape")
    if kind == PRE_ADD_RMSNORM and (norm_weight is None or norm_weight.numel() != n_in_features):
        raise ValueError("matmul_matgptq_prologue: the norm needs a weight of n_in_features elements")
    y = torch.empty((rows, n_out_features), dtype=torch.float16, device=a.device)
    ptr = lambda t: None if t is None else t.data_ptr()
    with torch.cuda.device(a.device):
        _lib.check(_lib.load().matgptq_gemm_prologue(
            bitwidth, group_size, n_out_features, n_in_features, rows, matgptq_weights.data_ptr(),
            matgptq_scales.data_ptr(), ptr(matgptq_zeros), kind, a.data_ptr(), ptr(added), ptr(norm_weight),
            ptr(residual_out), eps, y.data_ptr(), torch.cuda.current_stream().cuda_stream, 1))
    return y
