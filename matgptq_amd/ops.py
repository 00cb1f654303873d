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
