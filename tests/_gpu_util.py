"""Helpers of the GPU tests: device buffers through torch, calls through the C ABI."""
from __future__ import annotations

import numpy as np
import torch

from matgptq_amd import _lib
from oracle import matgptq_oracle as o

DEV = "cuda:0"
# Acceptance rule of the task statement: max rel err <= 1e-2 against the oracle (fp32
# accumulate).  "Relative" is taken against the largest output of the call; in addition
# every element must be within 1e-2 of its own value plus a rounding allowance tied to
# the size of the dot product, sum_k |w||x| (the quantity rounding errors scale with).
REL_TOL = 1e-2
BOUND_TOL = 1e-3
# Regression bound next to the acceptance rule: the kernels measure 3e-4 .. 6e-4 of the largest
# output (one fp16 rounding of the result is 4.9e-4 of its own value); a kernel that lost part of
# a group would still pass 1e-2 on many shapes, it would not pass this.
REGRESSION_TOL = 2e-3


def lib():
    return _lib.load()


def stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def to_dev(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def pack_device(codes: np.ndarray, bits: int, from_master: bool) -> torch.Tensor:
    n, k = codes.shape
    c = to_dev(codes)
    out = torch.empty(lib().matgptq_packed_words(bits, n, k), dtype=torch.int32, device=DEV)
    _lib.check(lib().matgptq_pack_device(c.data_ptr(), n, k, bits, int(from_master), out.data_ptr(), stream()))
    return out


def reorder_device(s: np.ndarray, n: int, k: int, g: int) -> torch.Tensor:
    src = to_dev(s)
    out = torch.empty_like(src)
    _lib.check(lib().matgptq_reorder_scales_device(src.data_ptr(), n, k, g, out.data_ptr(), stream()))
    return out


def gemm(bits, g, n, k, x: torch.Tensor, packed, scales, zeros=None, flags=1) -> torch.Tensor:
    m = x.shape[0]
    # poisoned: the caching allocator hands back the block of the previous call, whose contents
    # would otherwise stand in for outputs a kernel failed to write
    y = torch.full((m, n), float("nan"), dtype=torch.float16, device=DEV)
    _lib.check(lib().matgptq_gemm(bits, g, n, k, m, packed.data_ptr(), scales.data_ptr(),
                                  zeros.data_ptr() if zeros is not None else None,
                                  x.data_ptr(), y.data_ptr(), stream(), flags))
    return y


class Layer:
    """A synthetic layer on the device together with its oracle weight."""

    def __init__(self, n, k, bits, g=128, seed=0, zero_points=True):
        self.n, self.k, self.bits, self.g = n, k, bits, g
        self.q, self.s, self.z = o.make_layer(n, k, g, seed=seed, symmetric=not zero_points)
        self.packed = pack_device(self.q, bits, from_master=True)
        self.scales = reorder_device(self.s, n, k, g)
        self.zeros = reorder_device(self.z, n, k, g) if zero_points else None
        self.w = o.dequantize(self.q, self.s, self.z, bits, g)  # oracle weight, fp16

    def run(self, x: np.ndarray, flags=1) -> np.ndarray:
        y = gemm(self.bits, self.g, self.n, self.k, to_dev(x), self.packed, self.scales, self.zeros, flags)
        torch.cuda.synchronize()
        return y.cpu().numpy()


def assert_close_to_oracle(y: np.ndarray, x: np.ndarray, w: np.ndarray, what=""):
    ref = o.linear_f64(x, w)
    bound = o.abs_product_bound(x, w)
    err = np.abs(y.astype(np.float64) - ref)
    scale = np.max(np.abs(ref))
    assert np.all(np.isfinite(y)), what
    assert err.max() <= REL_TOL * scale, f"{what}: max err {err.max():.3e} vs {REL_TOL} * {scale:.3e}"
    allowed = REL_TOL * np.abs(ref) + BOUND_TOL * bound
    worst = np.max(err - allowed)
    assert worst <= 0, f"{what}: element-wise excess {worst:.3e}"


def assert_regression_bound(y: np.ndarray, x: np.ndarray, w: np.ndarray, what=""):
    ref = o.linear_f64(x, w)
    err = np.max(np.abs(y.astype(np.float64) - ref))
    assert err <= REGRESSION_TOL * np.max(np.abs(ref)), f"{what}: max err {err:.3e} above the regression bound"


def oracle_product_in_chunks(q, s, z, bits, g, x, rows_per_chunk=4096):
    """float64 product of `x` with the oracle weight and the bound sum |w||x|, formed over chunks
    of weight rows so that a layer of several hundred million weights needs little memory."""
    n = q.shape[0]
    ref = np.empty((x.shape[0], n), dtype=np.float64)
    bound = np.empty_like(ref)
    for r0 in range(0, n, rows_per_chunk):
        r1 = min(n, r0 + rows_per_chunk)
        w = o.dequantize(q[r0:r1], s[r0:r1], z[r0:r1], bits, g)
        ref[:, r0:r1] = o.linear_f64(x, w)
        bound[:, r0:r1] = o.abs_product_bound(x, w)
    return ref, bound


def assert_close_to_reference(y: np.ndarray, ref: np.ndarray, bound: np.ndarray, what="", regression=True):
    err = np.abs(y.astype(np.float64) - ref)
    scale = np.max(np.abs(ref))
    assert np.all(np.isfinite(y)), what
    assert err.max() <= REL_TOL * scale, f"{what}: max err {err.max():.3e} vs {REL_TOL} * {scale:.3e}"
    worst = np.max(err - (REL_TOL * np.abs(ref) + BOUND_TOL * bound))
    assert worst <= 0, f"{what}: element-wise excess {worst:.3e}"
    if regression:
        assert err.max() <= REGRESSION_TOL * scale, f"{what}: max err {err.max():.3e} above the regression bound"
