"""MI355X (gfx950) implementation of MatGPTQ's bit-sliced mixed-precision GEMM.

Importing this package loads the PyTorch extension `matgptq_amd/lib/_C.so` (which
links the C ABI library `libmatgptq_hip.so`) and thereby registers

    torch.ops.matgptq_cuda.pack_matgptq_qweights
    torch.ops.matgptq_cuda.reorder_matgptq_scales
    torch.ops.matgptq_cuda.matmul_matgptq

with the schemas of the reference (inference_lib/matgptq_cuda/csrc/bindings.cpp:198-200)
plus the additive ops documented in `matgptq_amd.ops`.  There is no fallback: when
the libraries have not been built (`python matgptq_amd/_build.py`), the import fails.
"""
from __future__ import annotations

import importlib.machinery
import importlib.util
import os
import sys

from . import _lib

_HERE = os.path.dirname(os.path.abspath(__file__))
_EXT_PATH = os.path.join(_HERE, "lib", "_C.so")

__all__ = ["_C", "ops", "load_extension", "matryoshka_slice"]


def load_extension():
    """Imports the extension module (idempotent) and returns it."""
    name = "matgptq_amd._C"
    if name in sys.modules:
        return sys.modules[name]
    if not os.path.exists(_EXT_PATH) or not os.path.exists(_lib.ABI_PATH):
        raise ImportError(
            f"{_EXT_PATH} / {_lib.ABI_PATH} not built: run `python matgptq_amd/_build.py` "
            "(hipcc --offload-arch=gfx950); the HIP path has no fallback")
    import torch  # noqa: F401  (libtorch must be loaded before the extension)

    loader = importlib.machinery.ExtensionFileLoader(name, _EXT_PATH)
    spec = importlib.util.spec_from_loader(name, loader)
    mod = importlib.util.module_from_spec(spec)
    loader.exec_module(mod)
    sys.modules[name] = mod
    return mod


_C = load_extension()

from . import ops  # noqa: E402  (registers the fake/meta implementations)
from .ops import matryoshka_slice  # noqa: E402
