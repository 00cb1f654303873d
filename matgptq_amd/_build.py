"""In-tree build of the native libraries (hipcc cross-compiles gfx950 without a GPU).

  libmatgptq_hip.so   the C ABI (include/matgptq_abi.h): HIP kernels + host packers
  libmatgptq_glue.so  decode-time operators between the linears (include/matgptq_glue.h)
  _C.so               the PyTorch extension that registers the torch ops on top of it

Both land in `matgptq_amd/lib/` so that a source snapshot carries them along.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(HERE, "lib", "obj")
ABI_SO = os.path.join(LIBDIR, "libmatgptq_hip.so")
TORCH_SO = os.path.join(LIBDIR, "_C.so")
GLUE_SO = os.path.join(LIBDIR, "libmatgptq_glue.so")

BITS = (2, 3, 4, 6, 8)
ARCH = "gfx950"

HIP_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    # packed fp32 VALU ops are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the native libraries cannot be built")
    return exe


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + r.stdout)
    return r.stdout


def _abi_jobs():
    hipcc = _hipcc()
    jobs = []
    # the GEMM kernels are built once per bitwidth and storage type (fp16, bf16); the
    # longest compilations go first so that the pool finishes evenly
    for stem in ("prefill_gfx950", "decode_gfx950", "skinny_gfx950", "gemv_gfx950"):
        for bf16 in (0, 1):
            for b in BITS:
                obj = os.path.join(OBJDIR, f"{stem}_b{b}{'_bf16' if bf16 else ''}.o")
                jobs.append((obj, [hipcc, *HIP_FLAGS, f"-DMATGPTQ_BITS={b}", f"-DMATGPTQ_BF16={bf16}", "-c",
                                   os.path.join(CSRC, stem + ".hip"), "-o", obj]))
    for stem in ("aux_gfx950", "abi"):
        obj = os.path.join(OBJDIR, stem + ".o")
        jobs.append((obj, [hipcc, *HIP_FLAGS, "-c", os.path.join(CSRC, stem + ".hip"), "-o", obj]))
    obj = os.path.join(OBJDIR, "pack_host.o")
    jobs.append((obj, ["g++", "-O3", "-std=c++17", "-fPIC", "-fopenmp", "-c",
                       os.path.join(CSRC, "pack_host.cpp"), "-o", obj]))
    return jobs


def build_abi(jobs: int = 8, verbose: bool = False) -> str:
    os.makedirs(OBJDIR, exist_ok=True)
    work = _abi_jobs()
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        outs = list(pool.map(lambda j: _run(j[1]), work))
    if verbose:
        for o in outs:
            if o.strip():
                print(o)
    objs = [w[0] for w in work]
    _run([_hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-fno-gpu-rdc", *objs,
          "-o", ABI_SO, "-fopenmp", "-Wno-unused-command-line-argument"])
    return ABI_SO


def build_torch_ext(verbose: bool = False) -> str:
    """Compiles torch_binding.cpp with the host compiler against libtorch and links
    it to libmatgptq_hip.so (found at run time through $ORIGIN)."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension as ce

    if not os.path.exists(ABI_SO):
        build_abi()
    inc = []
    for p in ce.include_paths("cuda"):
        inc += ["-isystem", p]
    inc += ["-isystem", sysconfig.get_paths()["include"]]
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    abi_flag = f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}"
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", abi_flag,
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_C",
           "-DTORCH_API_INCLUDE_EXTENSION_H", *inc,
           os.path.join(CSRC, "torch_binding.cpp"), "-o", TORCH_SO,
           f"-L{LIBDIR}", "-lmatgptq_hip", f"-L{torch_lib}", "-lc10", "-ltorch", "-ltorch_cpu",
           "-ltorch_python", "-lc10_hip", "-ltorch_hip", "-L/opt/rocm/lib", "-lamdhip64",
           "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}", "-Wl,-rpath,/opt/rocm/lib",
           "-Wno-deprecated-declarations"]
    out = _run(cmd)
    if verbose and out.strip():
        print(out)
    return TORCH_SO


def build_glue(verbose: bool = False) -> str:
    os.makedirs(LIBDIR, exist_ok=True)
    out = _run([_hipcc(), *HIP_FLAGS, "-shared", os.path.join(CSRC, "glue_gfx950.hip"), "-o", GLUE_SO])
    if verbose and out.strip():
        print(out)
    return GLUE_SO


def build_all(verbose: bool = False) -> None:
    build_abi(verbose=verbose)
    build_glue(verbose=verbose)
    build_torch_ext(verbose=verbose)


if __name__ == "__main__":
    build_all(verbose="-v" in sys.argv)
    print("built", ABI_SO, TORCH_SO)
