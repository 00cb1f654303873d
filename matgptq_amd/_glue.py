"""ctypes face of the decode-time operators between the linears (include/matgptq_glue.h).

Loaded from `matgptq_amd/lib/libmatgptq_glue.so`, built by `matgptq_amd._build.build_glue()`.
The functions below take torch tensors on the GPU, launch on torch's current stream and
return nothing: outputs are written into the tensors passed in.  There is no fallback:
a missing library raises.
"""
from __future__ import annotations

import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
GLUE_PATH = os.path.join(_HERE, "lib", "libmatgptq_glue.so")
MAX_CONTEXT = 8192

EXPORTS = ("matgptq_glue_strerror", "matgptq_glue_add_rmsnorm", "matgptq_glue_rope_cache",
           "matgptq_glue_attention", "matgptq_glue_rope_attention", "matgptq_glue_attention_workspace_floats",
           "matgptq_glue_attention_split", "matgptq_glue_silu_mul", "matgptq_glue_argmax")

_lib = None


class GlueError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(GLUE_PATH):
        raise GlueError(f"{GLUE_PATH} is missing: build it with `python matgptq_amd/_build.py`; "
                        "there is no fallback path")
    L = ctypes.CDLL(GLUE_PATH)
    vp, i64, ci, f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
    L.matgptq_glue_strerror.argtypes = [ci]
    L.matgptq_glue_strerror.restype = ctypes.c_char_p
    L.matgptq_glue_add_rmsnorm.argtypes = [vp, vp, vp, vp, i64, i64, f32, vp]
    L.matgptq_glue_rope_cache.argtypes = [vp, vp, vp, vp, vp, vp, i64, ci, ci, ci, i64, vp]
    L.matgptq_glue_attention.argtypes = [vp, vp, vp, vp, vp, i64, ci, ci, ci, i64, vp]
    L.matgptq_glue_rope_attention.argtypes = [vp, vp, vp, vp, vp, vp, vp, ci, ci, ci, i64, vp]
    L.matgptq_glue_silu_mul.argtypes = [vp, vp, i64, i64, vp]
    L.matgptq_glue_argmax.argtypes = [vp, vp, i64, i64, vp]
    L.matgptq_glue_attention_split.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, i64, ci, ci, ci, i64, ci, vp]
    L.matgptq_glue_attention_workspace_floats.argtypes = [i64, ci, i64]
    for name in EXPORTS[1:]:
        getattr(L, name).restype = ci
    L.matgptq_glue_attention_workspace_floats.restype = ctypes.c_size_t
    _lib = L
    return L


def _check(code: int) -> None:
    if code != 0:
        raise GlueError(load().matgptq_glue_strerror(code).decode())


def _f16(*tensors) -> None:
    for t in tensors:
        if t is not None and (t.dtype != torch.float16 or not t.is_cuda or not t.is_contiguous()):
            raise GlueError("expected contiguous float16 tensors on the GPU")


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def add_rmsnorm(h, delta, weight, x, eps: float) -> None:
    """h += delta (if not None); x = rms_norm(h) * weight.  h, delta, x: [M, H]."""
    _f16(h, delta, weight, x)
    m, hidden = h.shape
    if x.shape != h.shape or weight.numel() != hidden or (delta is not None and delta.shape != h.shape):
        raise GlueError("add_rmsnorm: shapes differ")
    _check(load().matgptq_glue_add_rmsnorm(h.data_ptr(), None if delta is None else delta.data_ptr(),
                                           weight.data_ptr(), x.data_ptr(), m, hidden, eps, _stream()))


def _pos_ok(pos, m: int) -> None:
    if pos.dtype != torch.int64 or not pos.is_cuda or not pos.is_contiguous() or pos.numel() != m:
        raise GlueError("pos must be a contiguous int64 tensor on the GPU with one entry per row")


def rope_cache(qkv, cos, sin, pos, k_cache, v_cache, heads: int, kv_heads: int) -> None:
    """Rotates the query heads of qkv [M, (heads + 2 kv_heads) * d] in place and writes rotated keys
    and the values into row pos[m] of k_cache / v_cache [kv_heads, max_ctx, d]."""
    _f16(qkv, cos, sin, k_cache, v_cache)
    m = qkv.shape[0]
    _pos_ok(pos, m)
    kv, max_ctx, d = k_cache.shape
    if (kv != kv_heads or v_cache.shape != k_cache.shape or qkv.shape[1] != (heads + 2 * kv_heads) * d
            or cos.shape != (max_ctx, d) or sin.shape != (max_ctx, d)):
        raise GlueError("rope_cache: shapes differ")
    _check(load().matgptq_glue_rope_cache(qkv.data_ptr(), cos.data_ptr(), sin.data_ptr(), pos.data_ptr(),
                                          k_cache.data_ptr(), v_cache.data_ptr(), m, heads, kv_heads, d, max_ctx,
                                          _stream()))


def attention(qkv, k_cache, v_cache, pos, out, heads: int, kv_heads: int) -> None:
    """out[M, heads * d] = attention of the query heads in qkv over cache rows 0 .. pos[m]."""
    _f16(qkv, k_cache, v_cache, out)
    m = qkv.shape[0]
    _pos_ok(pos, m)
    kv, max_ctx, d = k_cache.shape
    if (kv != kv_heads or v_cache.shape != k_cache.shape or qkv.shape[1] != (heads + 2 * kv_heads) * d
            or out.shape != (m, heads * d)):
        raise GlueError("attention: shapes differ")
    _check(load().matgptq_glue_attention(qkv.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), pos.data_ptr(),
                                         out.data_ptr(), m, heads, kv_heads, d, max_ctx, _stream()))


def rope_attention(qkv, cos, sin, pos, k_cache, v_cache, out, heads: int, kv_heads: int) -> None:
    """`rope_cache` and `attention` for one row in one launch (same results; qkv is left as it is)."""
    _f16(qkv, cos, sin, k_cache, v_cache, out)
    _pos_ok(pos, 1)
    kv, max_ctx, d = k_cache.shape
    if (qkv.shape[0] != 1 or kv != kv_heads or v_cache.shape != k_cache.shape
            or qkv.shape[1] != (heads + 2 * kv_heads) * d or cos.shape != (max_ctx, d) or sin.shape != (max_ctx, d)
            or out.shape != (1, heads * d)):
        raise GlueError("rope_attention: shapes differ")
    _check(load().matgptq_glue_rope_attention(qkv.data_ptr(), cos.data_ptr(), sin.data_ptr(), pos.data_ptr(),
                                              k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), heads,
                                              kv_heads, d, max_ctx, _stream()))


def attention_workspace(rows: int, heads: int, max_ctx: int, device):
    """Workspace of `attention_split` for up to `rows` query rows (contents irrelevant)."""
    floats = load().matgptq_glue_attention_workspace_floats(rows, heads, max_ctx)
    return torch.empty(floats, dtype=torch.float32, device=device)


def attention_split(qkv, cos, sin, pos, k_cache, v_cache, out, workspace, heads: int, kv_heads: int,
                    fuse_rotary: bool) -> None:
    """`attention` with the context split over workgroups; with `fuse_rotary` (one row) also the
    rotary embedding and the cache write, like `rope_attention`."""
    _f16(qkv, k_cache, v_cache, out, *((cos, sin) if fuse_rotary else ()))
    m = qkv.shape[0]
    _pos_ok(pos, m)
    kv, max_ctx, d = k_cache.shape
    if (kv != kv_heads or v_cache.shape != k_cache.shape or qkv.shape[1] != (heads + 2 * kv_heads) * d
            or out.shape != (m, heads * d) or (fuse_rotary and (cos.shape != (max_ctx, d) or sin.shape != (max_ctx, d)))):
        raise GlueError("attention_split: shapes differ")
    need = load().matgptq_glue_attention_workspace_floats(m, heads, max_ctx)
    if (workspace.dtype != torch.float32 or not workspace.is_cuda or not workspace.is_contiguous()
            or workspace.numel() < need):
        raise GlueError("attention_split: workspace too small or of the wrong type")
    _check(load().matgptq_glue_attention_split(
        qkv.data_ptr(), cos.data_ptr() if fuse_rotary else None, sin.data_ptr() if fuse_rotary else None,
        pos.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), workspace.data_ptr(),
        m, heads, kv_heads, d, max_ctx, int(fuse_rotary), _stream()))


def silu_mul(gate_up, out) -> None:
    """out[M, F] = silu(gate_up[:, :F]) * gate_up[:, F:]."""
    _f16(gate_up, out)
    m, f = out.shape
    if gate_up.shape != (m, 2 * f):
        raise GlueError("silu_mul: shapes differ")
    _check(load().matgptq_glue_silu_mul(gate_up.data_ptr(), out.data_ptr(), m, f, _stream()))


def argmax(x, out) -> None:
    """out[m] = torch.argmax(x[m]) for fp32 rows x [M, n]; `out` int64 [M]."""
    if (x.dtype != torch.float32 or out.dtype != torch.int64 or not x.is_cuda or not out.is_cuda
            or not x.is_contiguous() or not out.is_contiguous() or x.dim() != 2 or out.shape != (x.shape[0],)):
        raise GlueError("argmax: fp32 [M, n] in, int64 [M] out, contiguous, on the GPU")
    _check(load().matgptq_glue_argmax(x.data_ptr(), out.data_ptr(), x.shape[0], x.shape[1], _stream()))
