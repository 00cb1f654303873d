"""ctypes face of the C ABI (include/matgptq_abi.h).

The library is loaded from `matgptq_amd/lib/libmatgptq_hip.so`; it is built by
`matgptq_amd._build.build_abi()` (or `__graft_entry__.build()`).  There is no
fallback: when the library is missing, loading raises.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
ABI_PATH = os.path.join(_HERE, "lib", "libmatgptq_hip.so")

FLAG_ASYNC = 1
FLAG_BF16 = 2
VARIANT_SHIFT = 8

EXPORTS = (
    "matgptq_abi_version", "matgptq_strerror", "matgptq_packed_words", "matgptq_gemm", "matgptq_gemm_prologue",
    "matgptq_pack_host", "matgptq_unpack_host", "matgptq_reorder_scales_host",
    "matgptq_pack_device", "matgptq_unpack_device", "matgptq_reorder_scales_device",
    "matgptq_slice_device", "matgptq_dequantize_device", "matgptq_describe_plan",
    "matgptq_master_words", "matgptq_pack_master_host", "matgptq_pack_master_device",
    "matgptq_unpack_master_host", "matgptq_unpack_master_device",
    "matgptq_gemm_master_workspace_bytes", "matgptq_gemm_master", "matgptq_gemm_master_static",
    "matgptq_probe_read",
)

_lib = None


class MatGPTQError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(ABI_PATH):
        raise MatGPTQError(
            f"{ABI_PATH} is missing: build it with `python matgptq_amd/_build.py` "
            "(hipcc, --offload-arch=gfx950); there is no fallback path")
    L = ctypes.CDLL(ABI_PATH)
    vp, i64, ci, u32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_uint32
    L.matgptq_abi_version.restype = ci
    L.matgptq_strerror.argtypes = [ci]
    L.matgptq_strerror.restype = ctypes.c_char_p
    L.matgptq_packed_words.argtypes = [ci, i64, i64]
    L.matgptq_packed_words.restype = ctypes.c_size_t
    L.matgptq_gemm.argtypes = [ci, ci, i64, i64, i64, vp, vp, vp, vp, vp, vp, u32]
    L.matgptq_gemm.restype = ci
    L.matgptq_gemm_prologue.argtypes = [ci, ci, i64, i64, i64, vp, vp, vp, ci, vp, vp, vp, vp, ctypes.c_float, vp, vp, u32]
    L.matgptq_gemm_prologue.restype = ci
    L.matgptq_pack_host.argtypes = [vp, i64, i64, ci, ci, vp]
    L.matgptq_pack_host.restype = ci
    L.matgptq_unpack_host.argtypes = [vp, i64, i64, ci, vp]
    L.matgptq_unpack_host.restype = ci
    L.matgptq_reorder_scales_host.argtypes = [vp, i64, i64, ci, vp]
    L.matgptq_reorder_scales_host.restype = ci
    L.matgptq_pack_device.argtypes = [vp, i64, i64, ci, ci, vp, vp]
    L.matgptq_pack_device.restype = ci
    L.matgptq_unpack_device.argtypes = [vp, i64, i64, ci, vp, vp]
    L.matgptq_unpack_device.restype = ci
    L.matgptq_reorder_scales_device.argtypes = [vp, i64, i64, ci, vp, vp]
    L.matgptq_reorder_scales_device.restype = ci
    L.matgptq_slice_device.argtypes = [vp, i64, ci, vp, vp]
    L.matgptq_slice_device.restype = ci
    L.matgptq_dequantize_device.argtypes = [ci, ci, i64, i64, vp, vp, vp, vp, vp]
    L.matgptq_dequantize_device.restype = ci
    L.matgptq_describe_plan.argtypes = [ci, ci, i64, i64, i64, ci, u32, ctypes.c_char_p,
                                        ctypes.c_size_t]
    L.matgptq_describe_plan.restype = ci
    L.matgptq_master_words.argtypes = [i64, i64]
    L.matgptq_master_words.restype = ctypes.c_size_t
    L.matgptq_pack_master_host.argtypes = [vp, i64, i64, vp]
    L.matgptq_pack_master_host.restype = ci
    L.matgptq_pack_master_device.argtypes = [vp, i64, i64, vp, vp]
    L.matgptq_pack_master_device.restype = ci
    L.matgptq_unpack_master_host.argtypes = [vp, i64, i64, ci, vp]
    L.matgptq_unpack_master_host.restype = ci
    L.matgptq_unpack_master_device.argtypes = [vp, i64, i64, ci, vp, vp]
    L.matgptq_unpack_master_device.restype = ci
    L.matgptq_gemm_master_workspace_bytes.argtypes = [ci, ci, i64, i64, i64, u32]
    L.matgptq_gemm_master_workspace_bytes.restype = ctypes.c_size_t
    L.matgptq_gemm_master.argtypes = [ci, ci, i64, i64, i64, vp, vp, vp, vp, vp, vp, ctypes.c_size_t, vp, u32]
    L.matgptq_gemm_master.restype = ci
    L.matgptq_gemm_master_static.argtypes = [ci, ci, i64, i64, i64, vp, vp, vp, vp, vp, vp, u32]
    L.matgptq_gemm_master_static.restype = ci
    L.matgptq_probe_read.argtypes = [vp, ctypes.c_size_t, vp]
    L.matgptq_probe_read.restype = ci
    _lib = L
    return L


def check(code: int) -> None:
    if code != 0:
        raise MatGPTQError(load().matgptq_strerror(code).decode())


def describe_plan(bits, group_size, n, k, m, has_zeros=False, flags=FLAG_ASYNC) -> str:
    buf = ctypes.create_string_buffer(128)
    check(load().matgptq_describe_plan(bits, group_size, n, k, m, int(has_zeros), flags, buf, 128))
    return buf.value.decode()
