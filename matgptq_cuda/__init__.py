"""Drop-in for the reference's `matgptq_cuda` package (inference_lib/matgptq_cuda/__init__.py).

Importing it registers `torch.ops.matgptq_cuda.{pack_matgptq_qweights,
reorder_matgptq_scales, matmul_matgptq}` - implemented by the gfx950 kernels of
`matgptq_amd` - and exposes the same three Python callables and the `_CUDA`
extension-module name the reference has.
"""
import sys as _sys

import matgptq_amd as _impl
from matgptq_amd.ops import (  # noqa: F401
    matmul_matgptq,
    matmul_matgptq_zp,
    pack_matgptq_master,
    pack_matgptq_qweights,
    reorder_matgptq_scales,
)

# the reference's pybind module lives at matgptq_cuda._CUDA (bindings.cpp:213-220)
_CUDA = _impl._C
_sys.modules[__name__ + "._CUDA"] = _CUDA
