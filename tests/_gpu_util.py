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
    y = torch.empty(m, n, dtype=torch.float16, device=DEV)
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
