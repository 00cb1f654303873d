"""Writes tests/golden/matgptq_golden.npz from the reference's own Python functions.

Run once in a container that has the reference checkout (it is not present on
the GPU box and is never needed there):

    python tests/golden/make_golden.py [/root/reference]

The reference ships no golden vectors for this path, and nothing in its test
suite pins `dequantize` / `FakeMatryoshkaLinear.forward` (its dtype promotion
of `uint8 - fp16` in particular), so the vectors below are produced by calling
those functions (src/quant_utils_matgpqt.py:9-22,174-224) on small seeded
inputs.  Only inputs and outputs are stored.
"""
from __future__ import annotations

import importlib.util
import os
import sys

import numpy as np
import torch

BITS = (2, 3, 4, 6, 8)


def load_reference_module(root: str):
    path = os.path.join(root, "src", "quant_utils_matgpqt.py")
    spec = importlib.util.spec_from_file_location("_ref_quant_utils_matgpqt", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def main() -> None:
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    ref = load_reference_module(root)
    out = {}

    # 1. slice table: every master code x every inference bitwidth
    q_all = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    out["slice_table"] = np.stack(
        [ref.matryoshka_slice(q_all, 8, b).numpy().astype(np.uint8) for b in BITS])

    # 2. dequantize on a small layer with real-valued scales and general zeros
    g = torch.Generator().manual_seed(1234)
    n, k, gs = 16, 256, 128
    q = torch.randint(0, 256, (n, k), generator=g, dtype=torch.uint8)
    scale = (torch.randn(n, k // gs, generator=g).abs() * 0.01 + 1e-3).to(torch.float16)
    zero = torch.randint(0, 256, (n, k // gs), generator=g).to(torch.float16)
    x = torch.randn(3, k, generator=g).to(torch.float16)
    out["q"] = q.numpy()
    out["scale"] = scale.numpy()
    out["zero"] = zero.numpy()
    out["x"] = x.numpy()
    for b in BITS:
        w = ref.dequantize(q.view(n, k // gs, gs), scale.view(n, -1, 1), zero.view(n, -1, 1), 8, b)
        out[f"w_b{b}"] = w.reshape(n, k).numpy()

    # 3. the module forward (get_weight + F.linear), CPU fp16
    for b in BITS:
        layer = _build_layer(ref, q, scale, zero, b)
        with torch.no_grad():
            y = layer(x)
        out[f"y_b{b}"] = y.numpy()

    # 4. group_size 32 and per-row (-1) variants of dequantize
    for gs2, tag in ((32, "g32"), (k, "gm1")):
        scale2 = (torch.randn(n, k // gs2, generator=g).abs() * 0.01 + 1e-3).to(torch.float16)
        zero2 = torch.randint(0, 256, (n, k // gs2), generator=g).to(torch.float16)
        out[f"scale_{tag}"] = scale2.numpy()
        out[f"zero_{tag}"] = zero2.numpy()
        w = ref.dequantize(q.view(n, k // gs2, gs2), scale2.view(n, -1, 1), zero2.view(n, -1, 1), 8, 3)
        out[f"w_b3_{tag}"] = w.reshape(n, k).numpy()

    # 5. the same functions on bfloat16 tensors (feature flag bit 1); values are stored as
    #    float32, which holds every bfloat16 exactly
    g5 = torch.Generator().manual_seed(4321)
    scale_bf = (torch.randn(n, k // gs, generator=g5).abs() * 0.01 + 1e-3).to(torch.bfloat16)
    zero_bf = torch.randint(0, 256, (n, k // gs), generator=g5).to(torch.bfloat16)
    x_bf = torch.randn(3, k, generator=g5).to(torch.bfloat16)
    out["scale_bf16"] = scale_bf.float().numpy()
    out["zero_bf16"] = zero_bf.float().numpy()
    out["x_bf16"] = x_bf.float().numpy()
    for b in BITS:
        w = ref.dequantize(q.view(n, k // gs, gs), scale_bf.view(n, -1, 1), zero_bf.view(n, -1, 1), 8, b)
        assert w.dtype == torch.bfloat16
        out[f"w_bf16_b{b}"] = w.reshape(n, k).float().numpy()
        layer = _build_layer(ref, q, scale_bf, zero_bf, b)
        with torch.no_grad():
            y = layer(x_bf)
        assert y.dtype == torch.bfloat16
        out[f"y_bf16_b{b}"] = y.float().numpy()

    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "matgptq_golden.npz")
    np.savez_compressed(dst, **out)
    print("wrote", dst, {k_: v.shape for k_, v in out.items()})


def _build_layer(ref, q, scale, zero, b):
    import inspect

    sig = inspect.signature(ref.FakeMatryoshkaLinear.__init__)
    kwargs = {}
    for name in list(sig.parameters)[1:]:
        if name == "qweight":
            kwargs[name] = q
        elif name == "scale":
            kwargs[name] = scale
        elif name == "zero":
            kwargs[name] = zero
        elif name == "master_bitwidth":
            kwargs[name] = 8
        elif name == "slice_bitwidth":
            kwargs[name] = b
        elif name in ("bias", "perm"):
            kwargs[name] = None
        else:
            raise RuntimeError(f"unexpected constructor argument {name}")
    return ref.FakeMatryoshkaLinear(**kwargs)


if __name__ == "__main__":
    main()
