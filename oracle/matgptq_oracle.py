"""CPU oracle for MatGPTQ's bit-sliced GEMM.  TEST INFRASTRUCTURE ONLY.

This module restates, in NumPy, the arithmetic of the reference's PyTorch
slice -> dequantize -> linear path.  It is the checker that the HIP kernels
are compared against; nothing in the shipped package may import it (only
`tests/`, `__graft_entry__.smoke()` and the `cpu_baseline` leg of `bench.py`).

Reference anchors (paths relative to the reference checkout):
  * matryoshka_slice      src/quant_utils_matgpqt.py:9-17
  * dequantize            src/quant_utils_matgpqt.py:19-22
  * FakeMatryoshkaLinear  src/quant_utils_matgpqt.py:202-224  (get_weight + forward)
  * kernel-form weights   inference_lib/test_matgptq_matmul.py:40
                          inference_lib/bench_matgptq_matmul.py:45
  * final scaling order   inference_lib/matgptq_cuda/csrc/matgptq_gemm.cu:615-632,943-949

How each function is pinned (see tests/test_oracle.py):
  * slice_codes      brute force over all 256 codes x {2,3,4,6,8} against the
                     independent closed form min(floor((q + 2^(7-b)) / 2^(8-b)), 2^b-1),
                     monotonicity, saturation, b == master identity, the C
                     restatement (oracle_c.c) and the committed golden table.
  * dequantize       exact integer identity (c << (8-b)) - z, single fp16
                     rounding of the product checked against float64 + one
                     rounding, z == 128 reduction to the kernel-form formula,
                     the committed golden vectors.
  * linear           float64 matmul of the fp16-rounded weight (library routine);
                     in the reference test's regime (0/1 scales, integer x) the
                     result is exact and is compared for equality.
  * bfloat16 forms   (round_to_bf16, dequantize_bf16, fake_matryoshka_linear_bf16)
                     rounding: exhaustive comparison with torch's float32 -> bfloat16
                     conversion on all 2^16 upper halves x three lower-half patterns
                     (tie, below, above); dequantize / forward: the committed golden
                     vectors the reference's dequantize and FakeMatryoshkaLinear give
                     on bfloat16 tensors.
"""
from __future__ import annotations

import numpy as np

SUPPORTED_BITS = (2, 3, 4, 6, 8)
SUPPORTED_GROUPS = (-1, 32, 128)
MASTER_BITS = 8


def slice_codes(q: np.ndarray, slice_bits: int, master_bits: int = MASTER_BITS) -> np.ndarray:
    """Rounded MSB slice of master codes (src/quant_utils_matgpqt.py:9-17).

    drop = 8 - slice_bits is hard-wired to an 8-bit store (:10).  When the slice
    equals the master width the code is returned as is (:13-14, the clamp is a
    no-op).  Otherwise the highest dropped bit is added as a rounding bit and the
    sum saturates at 2^b - 1 (:16-17).
    """
    q = np.asarray(q)
    if q.dtype != np.uint8:
        raise TypeError("master codes must be uint8")
    drop = 8 - slice_bits
    # torch computes on uint8; widen so that floor + round_bit cannot wrap.
    floor = (q.astype(np.int32) >> drop)
    top = (1 << slice_bits) - 1
    if master_bits == slice_bits:
        return np.clip(floor, 0, top).astype(np.uint8)
    round_bit = (q.astype(np.int32) >> (drop - 1)) & 1
    return np.clip(floor + round_bit, 0, top).astype(np.uint8)


def _expand_groups(a: np.ndarray, n: int, k: int, group_size: int) -> np.ndarray:
    """Broadcast a per-group [N, K/g] array to [N, K]."""
    g = k if group_size == -1 else group_size
    a = np.asarray(a).reshape(n, k // g)
    return np.repeat(a, g, axis=1)


def dequantize(q: np.ndarray, scale: np.ndarray, zero: np.ndarray, slice_bits: int,
               group_size: int, master_bits: int = MASTER_BITS,
               dtype=np.float16) -> np.ndarray:
    """W = scale * ((slice(q) << (master - b)) - zero)   (src/quant_utils_matgpqt.py:19-22).

    dtype flow as torch executes it on fp16 tensors: the shifted code is uint8,
    `q_shifted - zero` promotes to the float dtype (integers of magnitude <= 255
    minus an fp16 zero: one rounding, exact for integral zeros), and the product
    with `scale` is rounded once more to the float dtype.
    """
    n, k = q.shape
    s = slice_codes(q, slice_bits, master_bits).astype(np.int32) << (master_bits - slice_bits)
    z = _expand_groups(np.asarray(zero, dtype=dtype), n, k, group_size)
    sc = _expand_groups(np.asarray(scale, dtype=dtype), n, k, group_size)
    diff = (s.astype(np.float64) - z.astype(np.float64)).astype(dtype)
    return (sc.astype(np.float64) * diff.astype(np.float64)).astype(dtype)


def dequantize_kernel_form(codes: np.ndarray, scale: np.ndarray, bits: int, group_size: int,
                           dtype=np.float16) -> np.ndarray:
    """Kernel-test closed form for already sliced codes
    (inference_lib/test_matgptq_matmul.py:40):
        W = ((c - 2^(b-1)) * scale) * 2^(8-b)
    evaluated in the float dtype like the reference test does.
    """
    n, k = codes.shape
    sc = _expand_groups(np.asarray(scale, dtype=dtype), n, k, group_size)
    centred = (codes.astype(np.int32) - (1 << (bits - 1))).astype(dtype)
    w = (centred.astype(np.float64) * sc.astype(np.float64)).astype(dtype)
    return (w.astype(np.float64) * float(1 << (8 - bits))).astype(dtype)


def linear(x: np.ndarray, w: np.ndarray, out_dtype=np.float16) -> np.ndarray:
    """Y = X @ W^T with wide accumulation and one final rounding
    (F.linear at src/quant_utils_matgpqt.py:223; fp32 accumulate in the BLAS).
    float64 accumulation is used here so that the oracle is the mathematical
    value of the product of the fp16 operands, rounded once.
    """
    y = np.asarray(x, dtype=np.float64) @ np.asarray(w, dtype=np.float64).T
    return y.astype(out_dtype)


def linear_f64(x: np.ndarray, w: np.ndarray) -> np.ndarray:
    """Un-rounded float64 product, for error-budget computations in tests."""
    return np.asarray(x, dtype=np.float64) @ np.asarray(w, dtype=np.float64).T


def fake_matryoshka_linear(x: np.ndarray, q: np.ndarray, scale: np.ndarray, zero: np.ndarray,
                           slice_bits: int, group_size: int,
                           master_bits: int = MASTER_BITS) -> np.ndarray:
    """FakeMatryoshkaLinear.forward without perm/bias (src/quant_utils_matgpqt.py:202-224)."""
    return linear(x, dequantize(q, scale, zero, slice_bits, group_size, master_bits))


# --------------------------------------------------------------------------
# bfloat16 storage (feature flag bit 1 of the reference, common.cuh:78-86): the same
# formulas evaluated on bfloat16 tensors.  bfloat16 values are carried as float32 here.
# --------------------------------------------------------------------------

def round_to_bf16(a: np.ndarray) -> np.ndarray:
    """float -> nearest bfloat16 (ties to even), returned as float32."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    r = np.where(nan, 0x7FC00000, r).astype(np.uint32)
    return r.view(np.float32)


def bf16_bits(a: np.ndarray) -> np.ndarray:
    """bfloat16-representable float32 -> uint16 bit patterns."""
    return (np.ascontiguousarray(a, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16)


def bf16_from_bits(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def dequantize_bf16(q: np.ndarray, scale: np.ndarray, zero: np.ndarray, slice_bits: int,
                    group_size: int, master_bits: int = MASTER_BITS) -> np.ndarray:
    """`dequantize` on bfloat16 tensors (src/quant_utils_matgpqt.py:19-22): the difference
    `q_shifted - zero` and the product with `scale` are each rounded to bfloat16.
    `scale`, `zero`: bfloat16 values held in float32.  Returns float32 holding bfloat16."""
    n, k = q.shape
    s = slice_codes(q, slice_bits, master_bits).astype(np.int32) << (master_bits - slice_bits)
    z = _expand_groups(np.asarray(zero, dtype=np.float32), n, k, group_size)
    sc = _expand_groups(np.asarray(scale, dtype=np.float32), n, k, group_size)
    diff = round_to_bf16(s.astype(np.float64) - z.astype(np.float64))
    # an 8-bit by 8-bit significand product is exact in float32: one rounding to bfloat16
    return round_to_bf16(sc.astype(np.float32) * diff)


def fake_matryoshka_linear_bf16(x: np.ndarray, q: np.ndarray, scale: np.ndarray, zero: np.ndarray,
                                slice_bits: int, group_size: int,
                                master_bits: int = MASTER_BITS) -> np.ndarray:
    """FakeMatryoshkaLinear.forward on bfloat16 tensors: wide accumulation, one rounding."""
    w = dequantize_bf16(q, scale, zero, slice_bits, group_size, master_bits)
    return round_to_bf16(linear_f64(x, w))


def abs_product_bound(x: np.ndarray, w: np.ndarray) -> np.ndarray:
    """sum_k |x||w| per output: the natural scale of rounding error of a dot product."""
    return np.abs(np.asarray(x, dtype=np.float64)) @ np.abs(np.asarray(w, dtype=np.float64)).T


# --------------------------------------------------------------------------
# Synthetic inputs of the benchmark configurations (seeded, NumPy only)
# --------------------------------------------------------------------------

def make_layer(n: int, k: int, group_size: int = 128, seed: int = 0, symmetric: bool = False):
    """Master 8-bit codes uniform in [0,255], scale = |N(0,1)|*0.01 + 1e-3 (fp16),
    zero uniform in [0,255] (fp16) or 128 when `symmetric`."""
    rng = np.random.default_rng(seed)
    g = k if group_size == -1 else group_size
    q = rng.integers(0, 256, size=(n, k), dtype=np.uint8)
    scale = (np.abs(rng.standard_normal((n, k // g))) * 0.01 + 1e-3).astype(np.float16)
    if symmetric:
        zero = np.full((n, k // g), 128.0, dtype=np.float16)
    else:
        zero = rng.integers(0, 256, size=(n, k // g)).astype(np.float16)
    return q, scale, zero


def make_activations(m: int, k: int, seed: int = 0, outlier_frac: float = 0.0,
                     outlier_gain: float = 20.0) -> np.ndarray:
    """x ~ N(0,1) fp16; optionally a seeded fraction of channels scaled up."""
    rng = np.random.default_rng(seed + 7919)
    x = rng.standard_normal((m, k))
    if outlier_frac > 0.0:
        n_out = max(1, int(round(k * outlier_frac)))
        cols = rng.choice(k, size=n_out, replace=False)
        x[:, cols] *= outlier_gain
    return x.astype(np.float16)
