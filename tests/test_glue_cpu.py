"""The library of decode-time operators between the linears loads without a GPU, exports what its
header declares, and rejects bad arguments before anything is launched."""
import ctypes
import os
import re

from matgptq_amd import _glue

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_every_declared_symbol_is_exported():
    header = open(os.path.join(ROOT, "include", "matgptq_glue.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    names = set(re.findall(r"\b(matgptq_glue_[a-z_0-9]+)\s*\(", header))
    assert names == set(_glue.EXPORTS)
    lib = ctypes.CDLL(_glue.GLUE_PATH)
    for n in sorted(names):
        assert hasattr(lib, n), n
    limit = int(re.search(r"#define MATGPTQ_GLUE_MAX_CONTEXT (\d+)", header).group(1))
    assert limit == _glue.MAX_CONTEXT


def test_argument_checks_come_before_any_launch():
    L = _glue.load()
    one = ctypes.c_void_p(16)  # never dereferenced: every call below fails its checks first
    assert L.matgptq_glue_add_rmsnorm(None, None, one, one, 1, 256, 1e-5, None) == -4
    assert L.matgptq_glue_add_rmsnorm(one, None, one, one, 1, 260, 1e-5, None) == -3
    assert L.matgptq_glue_add_rmsnorm(one, None, one, one, 1, 16384, 1e-5, None) == -8
    assert L.matgptq_glue_rope_cache(one, one, one, None, one, one, 1, 4, 2, 128, 64, None) == -4
    assert L.matgptq_glue_rope_cache(one, one, one, one, one, one, 1, 4, 3, 128, 64, None) == -3
    assert L.matgptq_glue_attention(one, one, one, one, one, 1, 4, 2, 64, 64, None) == -3
    assert L.matgptq_glue_attention(one, one, one, one, one, 1, 4, 2, 128, _glue.MAX_CONTEXT + 1, None) == -8
    assert L.matgptq_glue_rope_attention(one, one, one, one, one, one, None, 4, 2, 128, 64, None) == -4
    assert L.matgptq_glue_rope_attention(one, one, one, one, one, one, one, 4, 2, 64, 64, None) == -3
    assert L.matgptq_glue_attention_split(one, None, None, one, one, one, one, None, 1, 4, 2, 128, 64, 0, None) == -4
    assert L.matgptq_glue_attention_split(one, None, None, one, one, one, one, one, 1, 4, 2, 128, 64, 1, None) == -4
    assert L.matgptq_glue_attention_split(one, one, one, one, one, one, one, one, 2, 4, 2, 128, 64, 1, None) == -3
    assert L.matgptq_glue_attention_split(one, None, None, one, one, one, one, one, 1, 6, 2, 128, 64, 0, None) == -3
    assert L.matgptq_glue_attention_workspace_floats(2, 4, 65) == 2 * 4 * 2 * 130
    assert L.matgptq_glue_argmax(None, one, 1, 8, None) == -4
    assert L.matgptq_glue_argmax(one, one, 0, 8, None) == -3
    assert L.matgptq_glue_argmax(one, one, 1, 2 ** 31, None) == -8
    assert L.matgptq_glue_silu_mul(one, None, 1, 64, None) == -4
    assert L.matgptq_glue_silu_mul(one, one, 1, 60, None) == -3
    assert b"NULL" in L.matgptq_glue_strerror(-4)
