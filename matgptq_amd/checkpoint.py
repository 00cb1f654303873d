"""Packed-checkpoint writer and reader of the `matgptq_quant` format.

Format (what the reference's `pack_quantized_model.py` writes and its vLLM plugin reads):

  * safetensors shards with the model's own tensor names, where every quantised linear
    `<layer>.weight` is replaced by `<layer>.qweight` (uint8 master codes `[N, K]`) and
    `<layer>.scales` (`[N, K/group]`, float16 or bfloat16)   (pack_quantized_model.py:79-91,112-117);
  * `model.safetensors.index.json` with the new weight map for sharded models (:96-98);
  * `config.json` whose `quantization_config` holds `group_size`, `modules_to_not_convert`,
    `master_bitwidth`, `inference_bitwidth`, `quant_method: "matgptq_quant"`, `quant_dtype`
    (:134-141); generation config and tokenizer files are carried over.

The quantiser's output that goes in is one directory per layer with a `data.pt` holding
`qweight` and `scale` (:11-22).  Additions, all optional:
  * `<layer>.zeros` when `data.pt` has a `zero` that is not 128 everywhere (asymmetric
    quantisation; the reference's packer drops `zero`, :15-18, and its kernels assume 128).
    `quantization_config.has_zeros` is then true and the plugin of this package registers a
    `zeros` parameter for every quantised linear; a checkpoint whose zeros are all 128 carries
    no such tensors and stays readable by the reference's plugin;
  * `<layer>.perm` when `data.pt` has a `perm` that is not the identity (act-order column
    permutation, src/mat_gptq.py:155-159); `quantization_config.has_perm` is then true;
  * a `layer_bitwidths` map in `quantization_config` (Mix'n'Match: the per-layer file of
    inference_demo_transformers.py:58-62 as part of the checkpoint).

Unlike the reference script this one needs neither `transformers` nor the model class:
`config.json` is edited as JSON and the tokenizer files are copied.  `data.pt` files are
loaded with `weights_only=True`.

    python -m matgptq_amd.checkpoint --model_name_or_path M --quantized_weights_path Q \\
        --packed_output_path OUT [--inference_bitwidth 4] [--master_bitwidth 8] \\
        [--group_size 128] [--quant_dtype float16] [--layer_bitwidths FILE]
"""
from __future__ import annotations

import argparse
import json
import os
import shutil
from typing import Dict, Iterator, Optional, Tuple

import torch
from safetensors import safe_open
from safetensors.torch import load_file, save_file

QUANT_METHOD = "matgptq_quant"
EXCLUDED = ("lm_head", "norm")  # pack_quantized_model.py:25-30
INDEX_NAME = "model.safetensors.index.json"
SINGLE_NAME = "model.safetensors"
# files a tokenizer / generation config consists of; copied when present
CARRIED_FILES = ("generation_config.json", "tokenizer.json", "tokenizer_config.json", "tokenizer.model",
                 "special_tokens_map.json", "added_tokens.json", "vocab.json", "merges.txt",
                 "chat_template.jinja")


def load_quantised_layer(layer_dir: str, mmap: bool = False) -> Dict[str, torch.Tensor]:
    """`qweight`, `scale` (and `zero`, `perm` when stored) of one layer (pack_quantized_model.py:11-22).
    With `mmap` the tensors are mapped from the file and read only where they are touched."""
    data_pt = os.path.join(layer_dir, "data.pt")
    if not os.path.exists(data_pt):
        raise FileNotFoundError(f"No data.pt found in {layer_dir}")
    data = torch.load(data_pt, map_location="cpu", weights_only=True, mmap=mmap)
    out = {"qweight": data["qweight"], "scale": data["scale"]}
    for key in ("zero", "perm"):
        if data.get(key) is not None:
            out[key] = data[key]
    return out


def should_skip_quantisation(module_name: str) -> bool:
    return any(excl in module_name for excl in EXCLUDED)


def read_layer_bitwidths(path: str) -> Dict[str, int]:
    """`layer_name: bitwidth` lines (inference_demo_transformers.py:58-62)."""
    out = {}
    with open(path, "r") as f:
        for line in f:
            if line.strip():
                name, bits = line.strip().split(":")
                out[name.strip()] = int(bits.strip())
    return out


def _check_layer(name: str, q: Dict[str, torch.Tensor], group_size: int, quant_dtype: torch.dtype):
    qw, sc = q["qweight"], q["scale"]
    if qw.dtype != torch.uint8 or qw.dim() != 2:
        raise ValueError(f"{name}: qweight must be a 2-D uint8 tensor")
    n, k = qw.shape
    groups = 1 if group_size == -1 else k // group_size
    if group_size != -1 and k % group_size != 0:
        raise ValueError(f"{name}: n_in_features must be divisible by group_size")
    if sc.numel() != n * groups:
        raise ValueError(f"{name}: scale has {sc.numel()} elements, expected {n * groups}")
    if "zero" in q and q["zero"].numel() != n * groups:
        raise ValueError(f"{name}: zero has {q['zero'].numel()} elements, expected {n * groups}")
    if "perm" in q and q["perm"].numel() != k:
        raise ValueError(f"{name}: perm must have n_in_features elements")
    del quant_dtype


def _packed_tensors(name: str, q: Dict[str, torch.Tensor], group_size: int,
                    quant_dtype: torch.dtype) -> Dict[str, torch.Tensor]:
    _check_layer(name, q, group_size, quant_dtype)
    n = q["qweight"].shape[0]
    out = {f"{name}.qweight": q["qweight"].cpu().contiguous(),
           f"{name}.scales": q["scale"].cpu().reshape(n, -1).contiguous()}
    if "zero" in q:
        out[f"{name}.zeros"] = q["zero"].cpu().reshape(n, -1).to(out[f"{name}.scales"].dtype).contiguous()
    if "perm" in q:
        out[f"{name}.perm"] = q["perm"].cpu().to(torch.int32).reshape(-1).contiguous()
    return out


def _all_symmetric(zero: torch.Tensor) -> bool:
    return bool((zero.float() == 128.0).all())


def _is_identity(perm: torch.Tensor) -> bool:
    perm = perm.reshape(-1).to(torch.int64)
    return bool((perm == torch.arange(perm.numel())).all())


def pack_model(model_name_or_path: str, quantised_dir: str, output_dir: str, group_size: int,
               master_bitwidth: int, inference_bitwidth: int, quant_dtype: str,
               layer_bitwidths: Optional[Dict[str, int]] = None) -> Dict[str, str]:
    """Writes the packed checkpoint; returns the new weight map (tensor name -> shard file).
    Same arguments as the reference's `pack_model` (pack_quantized_model.py:33-41) plus the
    optional per-layer bitwidth map."""
    if quant_dtype not in ("float16", "bfloat16"):
        raise ValueError("quant_dtype must be float16 or bfloat16")
    dtype = torch.float16 if quant_dtype == "float16" else torch.bfloat16
    os.makedirs(output_dir, exist_ok=True)
    index_path = os.path.join(model_name_or_path, INDEX_NAME)
    single_path = os.path.join(model_name_or_path, SINGLE_NAME)
    quantised_layers = {name for name in os.listdir(quantised_dir)
                        if os.path.isdir(os.path.join(quantised_dir, name))}
    new_weight_map: Dict[str, str] = {}
    if not os.path.exists(index_path) and not os.path.exists(single_path):
        raise FileNotFoundError(f"Neither {INDEX_NAME} nor {SINGLE_NAME} found.")
    # One rule for the whole checkpoint, because the plugin registers the same parameters for
    # every quantised linear: zeros are written for all layers or for none, and so is perm.
    packable = sorted(name for name in quantised_layers if not should_skip_quantisation(name))
    has_zeros = has_perm = False
    for layer in packable:
        q = load_quantised_layer(os.path.join(quantised_dir, layer), mmap=True)  # the codes stay on disk
        has_zeros = has_zeros or ("zero" in q and not _all_symmetric(q["zero"]))
        has_perm = has_perm or ("perm" in q and not _is_identity(q["perm"]))

    def convert(shard_name: str, names, tensors) -> None:
        new_tensors: Dict[str, torch.Tensor] = {}
        for t_name in names:
            tensor = tensors.get(t_name)
            if tensor is None:
                continue
            if t_name.endswith(".weight"):
                layer = t_name.rsplit(".", 1)[0]
                if layer in quantised_layers and not should_skip_quantisation(layer):
                    q = load_quantised_layer(os.path.join(quantised_dir, layer))
                    if has_zeros:
                        q.setdefault("zero", torch.full_like(q["scale"], 128.0))
                    else:
                        q.pop("zero", None)
                    if has_perm:
                        q.setdefault("perm", torch.arange(q["qweight"].shape[1]))
                    else:
                        q.pop("perm", None)
                    for key, value in _packed_tensors(layer, q, group_size, dtype).items():
                        new_tensors[key] = value
                        new_weight_map[key] = shard_name
                    continue
            new_tensors[t_name] = tensor
            new_weight_map[t_name] = shard_name
        save_file(new_tensors, os.path.join(output_dir, shard_name))

    if os.path.exists(index_path):
        with open(index_path, "r") as f:
            original_map: Dict[str, str] = json.load(f)["weight_map"]
        for shard_name in sorted(set(original_map.values())):
            tensors = load_file(os.path.join(model_name_or_path, shard_name))
            convert(shard_name, [t for t, s in original_map.items() if s == shard_name], tensors)
        with open(os.path.join(output_dir, INDEX_NAME), "w") as f:
            json.dump({"metadata": {}, "weight_map": new_weight_map}, f)
    else:
        tensors = load_file(single_path)
        convert(SINGLE_NAME, list(tensors.keys()), tensors)

    config_path = os.path.join(model_name_or_path, "config.json")
    config = {}
    if os.path.exists(config_path):
        with open(config_path, "r") as f:
            config = json.load(f)
    quantization_config = {
        "group_size": group_size,
        "modules_to_not_convert": list(EXCLUDED),
        "master_bitwidth": master_bitwidth,
        "inference_bitwidth": inference_bitwidth,
        "quant_method": QUANT_METHOD,
        "quant_dtype": quant_dtype,
    }
    if has_zeros:
        quantization_config["has_zeros"] = True
    if has_perm:
        quantization_config["has_perm"] = True
    if layer_bitwidths:
        quantization_config["layer_bitwidths"] = dict(layer_bitwidths)
    config["quantization_config"] = quantization_config
    with open(os.path.join(output_dir, "config.json"), "w") as f:
        json.dump(config, f, indent=2)
    for name in CARRIED_FILES:
        src = os.path.join(model_name_or_path, name)
        if os.path.exists(src):
            shutil.copyfile(src, os.path.join(output_dir, name))
    return new_weight_map


# ----------------------------------------------------------------------------- reader

def read_quantization_config(packed_dir: str) -> dict:
    with open(os.path.join(packed_dir, "config.json"), "r") as f:
        qc = json.load(f).get("quantization_config")
    if not qc or qc.get("quant_method") != QUANT_METHOD:
        raise ValueError(f"{packed_dir}: config.json has no {QUANT_METHOD} quantization_config")
    for key in ("group_size", "master_bitwidth", "inference_bitwidth", "quant_dtype"):
        if key not in qc:
            raise ValueError(f"{packed_dir}: quantization_config lacks {key}")
    return qc


def weight_map(packed_dir: str) -> Dict[str, str]:
    index_path = os.path.join(packed_dir, INDEX_NAME)
    if os.path.exists(index_path):
        with open(index_path, "r") as f:
            return json.load(f)["weight_map"]
    single = os.path.join(packed_dir, SINGLE_NAME)
    if not os.path.exists(single):
        raise FileNotFoundError(f"Neither {INDEX_NAME} nor {SINGLE_NAME} found.")
    with safe_open(single, framework="pt") as f:
        return {name: SINGLE_NAME for name in f.keys()}


def iter_quantised_layers(packed_dir: str) -> Iterator[Tuple[str, Dict[str, torch.Tensor]]]:
    """Yields `(layer_name, {"qweight", "scales", ["zeros"], ["perm"]})` for every quantised
    linear of a packed checkpoint, reading one tensor at a time."""
    wm = weight_map(packed_dir)
    layers = sorted(name[: -len(".qweight")] for name in wm if name.endswith(".qweight"))
    for layer in layers:
        out = {}
        for key in ("qweight", "scales", "zeros", "perm"):
            t_name = f"{layer}.{key}"
            if t_name in wm:
                with safe_open(os.path.join(packed_dir, wm[t_name]), framework="pt") as f:
                    out[key] = f.get_tensor(t_name)
        if "scales" not in out:
            raise ValueError(f"{layer}: qweight without scales")
        yield layer, out


def bitwidth_of(layer: str, quantization_config: dict) -> int:
    """Longest matching suffix of `layer_bitwidths`, else `inference_bitwidth` (the rule of
    the vLLM plugin of this package)."""
    best, best_len = quantization_config["inference_bitwidth"], -1
    for key, bits in (quantization_config.get("layer_bitwidths") or {}).items():
        if (layer == key or layer.endswith(key)) and len(key) > best_len:
            best, best_len = bits, len(key)
    return best


def build_linear(tensors: Dict[str, torch.Tensor], bitwidth: int, quantization_config: dict,
                 device: str = "cuda"):
    """A `MatGPTQLinear` for one layer of a packed checkpoint: slice to `bitwidth`, pack,
    reorder (inference_demo_transformers.py:30-40).  A stored column permutation becomes part
    of the module, which gathers its input features with it (`x[..., perm]`)."""
    from matgptq_cuda.matgptq_linear import MatGPTQLinear

    from .ops import matryoshka_slice

    master = quantization_config["master_bitwidth"]
    q = tensors["qweight"].to(device)
    zeros = tensors.get("zeros")
    perm = tensors.get("perm")
    return MatGPTQLinear(matryoshka_slice(q, master, bitwidth), tensors["scales"].to(device), bitwidth,
                         quantization_config["group_size"],
                         zeros=zeros.to(device) if zeros is not None else None,
                         perm=perm.to(device) if perm is not None else None)


def main() -> None:
    ap = argparse.ArgumentParser(description="Pack a quantised model into new safetensor shards")
    ap.add_argument("--model_name_or_path", type=str, required=True)
    ap.add_argument("--quantized_weights_path", type=str, required=True)
    ap.add_argument("--packed_output_path", type=str, required=True)
    ap.add_argument("--inference_bitwidth", type=int, default=4)
    ap.add_argument("--master_bitwidth", type=int, default=8)
    ap.add_argument("--group_size", type=int, default=128)
    ap.add_argument("--quant_dtype", type=str, default="float16", choices=["float16", "bfloat16"])
    ap.add_argument("--layer_bitwidths", type=str, default=None,
                    help="file of `layer_name: bitwidth` lines stored as quantization_config.layer_bitwidths")
    args = ap.parse_args()
    pack_model(args.model_name_or_path, args.quantized_weights_path, args.packed_output_path,
               args.group_size, args.master_bitwidth, args.inference_bitwidth, args.quant_dtype,
               read_layer_bitwidths(args.layer_bitwidths) if args.layer_bitwidths else None)


if __name__ == "__main__":
    main()
