"""vLLM quantization plugin `matgptq_quant` backed by the gfx950 kernels.

Same registry name, config keys, layer parameters and method names as the reference
plugin (inference_lib/vllm_matgptq.py:18-201):

    config.json "quantization_config": {quant_method: "matgptq_quant", group_size,
        master_bitwidth, inference_bitwidth, quant_dtype, modules_to_not_convert}
    layer parameters  qweight uint8 [N, K] (8-bit master codes), scales [N, K/group_size]

Differences, all additive:
  * the slice of the master codes is the package's own (`matgptq_amd.ops.matryoshka_slice`;
    the reference imports it from its calibration tree through a sys.path edit, :1-3,13);
  * slicing and packing happen on the GPU in one kernel when the master codes are
    already there (the reference copies them to the host and back);
  * optional key `layer_bitwidths` {prefix-suffix: bits} selects a bitwidth per layer
    (Mix'n'Match); layers not listed use `inference_bitwidth`;
  * optional keys `has_zeros` / `has_perm`: the checkpoint carries `<layer>.zeros`
    [N, K/group_size] (asymmetric quantisation) / `<layer>.perm` [K] (act-order) for every
    quantised linear, and `create_weights` registers parameters of those names so that the
    loader finds a destination for them.  Without the keys neither is registered, as in the
    reference.  vLLM is not importable in this build's environment: what its loader does with
    these parameters is exercised only through a stand-in loader in the tests;
  * `keep_master_codes` (constructor argument / config key, default false): the 8-bit master
    codes stay resident after loading next to the packed slice and `set_bitwidth` re-slices a
    layer in place (one device pass over its codes);
  * `resident_master_planes` (same, default false): ONLY the master codes stay resident, as bit
    planes (`pack_matgptq_master_resident`), and every product goes through
    `matmul_matgptq_master`, which slices to the layer's current bitwidth in registers:
    `set_bitwidth` then changes a number and moves nothing.

vLLM itself is imported lazily: without it the module still imports (the classes then
derive from small local bases), which is what the CPU test-suite exercises.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch
from torch.nn.parameter import Parameter

import matgptq_cuda  # noqa: F401  (registers torch.ops.matgptq_cuda.*)
from matgptq_amd.ops import matryoshka_slice
from matgptq_cuda.matgptq_linear import MatGTPQ_FeatureFlags

try:  # pragma: no cover - exercised only where vLLM is installed
    from vllm.model_executor.layers.linear import (LinearBase, LinearMethodBase,
                                                   UnquantizedLinearMethod)
    from vllm.model_executor.layers.quantization import register_quantization_config
    from vllm.model_executor.layers.quantization.base_config import (QuantizationConfig,
                                                                     QuantizeMethodBase)
    from vllm.model_executor.parameter import ModelWeightParameter
    from vllm.model_executor.utils import set_weight_attrs
    HAVE_VLLM = True
except ImportError:
    HAVE_VLLM = False

    class QuantizationConfig:  # minimal stand-ins so that the plugin logic is testable
        def __init__(self) -> None:
            pass

        @staticmethod
        def get_from_keys(config: dict, keys: List[str]):
            for k in keys:
                if k in config:
                    return config[k]
            raise ValueError(f"Cannot find any of {keys} in the model's quantization config.")

    class QuantizeMethodBase:
        pass

    class LinearMethodBase(QuantizeMethodBase):
        pass

    class LinearBase(torch.nn.Module):
        pass

    class UnquantizedLinearMethod(LinearMethodBase):
        pass

    def register_quantization_config(name: str):
        def deco(cls):
            return cls
        return deco

    def set_weight_attrs(weight: torch.Tensor, attrs: Optional[dict]) -> None:
        for k, v in (attrs or {}).items():
            setattr(weight, k, v)

    def ModelWeightParameter(data: torch.Tensor, input_dim: int, output_dim: int, weight_loader=None):
        p = Parameter(data, requires_grad=False)
        set_weight_attrs(p, {"input_dim": input_dim, "output_dim": output_dim,
                             "weight_loader": weight_loader})
        return p


@register_quantization_config("matgptq_quant")
class MatGPTQConfig(QuantizationConfig):
    """Quantization config (reference: inference_lib/vllm_matgptq.py:18-86)."""

    def __init__(
        self,
        group_size: int = 128,
        master_bitwidth: int = 8,
        inference_bitwidth: int = 4,
        quant_dtype: str = "float16",
        modules_to_not_convert: Optional[List[str]] = None,
        layer_bitwidths: Optional[Dict[str, int]] = None,
        has_zeros: bool = False,
        has_perm: bool = False,
        keep_master_codes: bool = False,
        resident_master_planes: bool = False,
    ) -> None:
        super().__init__()
        assert group_size in [-1, 32, 128]
        assert quant_dtype in ["float16", "bfloat16"]
        dtype_map = {"float16": torch.float16, "bfloat16": torch.bfloat16}

        self.group_size = group_size
        self.master_bitwidth = master_bitwidth
        self.inference_bitwidth = inference_bitwidth
        self.quant_dtype = dtype_map.get(quant_dtype, torch.float16)
        self.modules_to_not_convert = modules_to_not_convert
        self.layer_bitwidths = dict(layer_bitwidths or {})
        self.has_zeros = bool(has_zeros)
        self.has_perm = bool(has_perm)
        self.keep_master_codes = bool(keep_master_codes)
        self.resident_master_planes = bool(resident_master_planes)
        if self.resident_master_planes and master_bitwidth != 8:
            raise ValueError("resident_master_planes needs 8-bit master codes")
        for bits in [inference_bitwidth, *self.layer_bitwidths.values()]:
            if bits not in (2, 3, 4, 6, 8):
                raise ValueError("bitwidth must be one of {2, 3, 4, 6, 8}")

        self.flag = MatGTPQ_FeatureFlags.ASYNC + MatGTPQ_FeatureFlags.IS_BF16 * (self.quant_dtype == torch.bfloat16)

    def get_name(self) -> str:
        return "matgptq_quant"

    def get_supported_act_dtypes(self) -> list:
        return [torch.float16, torch.bfloat16]

    @classmethod
    def get_min_capability(cls) -> int:
        # An NVIDIA SM number in the reference (80); vLLM's ROCm platform reports the
        # gfx target as major*10+minor (gfx950 -> 95), which passes the same check.
        return 80

    @staticmethod
    def get_config_filenames() -> List[str]:
        return []

    @classmethod
    def from_config(cls, config: dict) -> "MatGPTQConfig":
        group_size = cls.get_from_keys(config, ["group_size"])
        master_bitwidth = cls.get_from_keys(config, ["master_bitwidth"])
        inference_bitwidth = cls.get_from_keys(config, ["inference_bitwidth"])
        modules_to_not_convert = cls.get_from_keys(config, ["modules_to_not_convert"])
        quant_dtype = cls.get_from_keys(config, ["quant_dtype"])
        layer_bitwidths = config.get("layer_bitwidths")
        return cls(group_size, master_bitwidth, inference_bitwidth, quant_dtype,
                   modules_to_not_convert, layer_bitwidths, config.get("has_zeros", False),
                   config.get("has_perm", False), config.get("keep_master_codes", False),
                   config.get("resident_master_planes", False))

    def bitwidth_for(self, prefix: str) -> int:
        """Bitwidth of the layer called `prefix`: the longest matching suffix key of
        `layer_bitwidths`, else `inference_bitwidth`."""
        best, best_len = self.inference_bitwidth, -1
        for key, bits in self.layer_bitwidths.items():
            if (prefix == key or prefix.endswith(key)) and len(key) > best_len:
                best, best_len = bits, len(key)
        return best

    def get_quant_method(self, layer: torch.nn.Module, prefix: str):
        if self.modules_to_not_convert is not None and any(
                prefix.endswith(module) for module in self.modules_to_not_convert):
            return UnquantizedLinearMethod()
        if isinstance(layer, LinearBase):
            return MatGPTQLinearMethod(self, self.bitwidth_for(prefix))
        return None


class MatGPTQLinearMethod(LinearMethodBase):
    """Linear method (reference: inference_lib/vllm_matgptq.py:89-201)."""

    def __init__(self, config: MatGPTQConfig, bitwidth: Optional[int] = None):
        super().__init__()
        self.config = config
        self.bitwidth = config.inference_bitwidth if bitwidth is None else bitwidth

    def create_weights(self, layer: torch.nn.Module, input_size_per_partition: int,
                       output_partition_sizes: List[int], input_size: int, output_size: int,
                       params_dtype: torch.dtype, **extra_weight_attrs):
        group = self.config.group_size if self.config.group_size != -1 else input_size_per_partition
        if input_size_per_partition % group != 0:
            raise ValueError(
                f"in_features per partition ({input_size_per_partition}) is not a multiple of the "
                f"quantisation group size ({group}); a tensor-parallel degree that splits K inside "
                "a group cannot be served")

        self.n_out_features = sum(output_partition_sizes)
        self.n_in_features = input_size_per_partition

        qweight = ModelWeightParameter(
            data=torch.empty(sum(output_partition_sizes), input_size_per_partition, dtype=torch.uint8),
            input_dim=1,
            output_dim=0,
            weight_loader=extra_weight_attrs.get("weight_loader"),
        )
        layer.register_parameter("qweight", qweight)

        scales = Parameter(
            torch.empty(self.n_out_features, input_size_per_partition // group,
                        dtype=self.config.quant_dtype),
            requires_grad=False,
        )
        set_weight_attrs(scales, {"input_dim": 1, "output_dim": 0, "packed_dim": 1, "pack_factor": 1}
                         | extra_weight_attrs)
        layer.register_parameter("scales", scales)

        if self.config.has_zeros:
            # same shape, sharding and loader as the scales; 128 wherever the loader writes nothing
            zeros = Parameter(torch.full_like(scales.data, 128.0), requires_grad=False)
            set_weight_attrs(zeros, {"input_dim": 1, "output_dim": 0, "packed_dim": 1, "pack_factor": 1}
                             | extra_weight_attrs)
            layer.register_parameter("zeros", zeros)
        if self.config.has_perm:
            if input_size_per_partition != input_size:
                raise ValueError(
                    "an act-order checkpoint (has_perm) permutes all input features of a layer; a "
                    "tensor-parallel degree that splits in_features cannot be served")
            perm = Parameter(torch.arange(input_size, dtype=torch.int32), requires_grad=False)
            set_weight_attrs(perm, {"input_dim": 0} | extra_weight_attrs)
            layer.register_parameter("perm", perm)

    def _pack_at(self, layer: torch.nn.Module, qweight: torch.Tensor, bitwidth: int) -> torch.Tensor:
        if qweight.is_cuda and self.config.master_bitwidth == 8:
            # slice and pack in one pass over the master codes, on the GPU
            return torch.ops.matgptq_cuda.pack_matgptq_master(
                qweight.contiguous(), self.n_out_features, self.n_in_features, bitwidth,
                self.config.group_size, self.config.flag)
        return torch.ops.matgptq_cuda.pack_matgptq_qweights(
            matryoshka_slice(qweight, self.config.master_bitwidth, bitwidth).contiguous(),
            self.n_out_features, self.n_in_features, bitwidth,
            self.config.group_size, self.config.flag)

    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        with torch.no_grad():
            qweight = layer.qweight.data
            if self.config.resident_master_planes:
                layer.matgptq_planes = Parameter(
                    torch.ops.matgptq_cuda.pack_matgptq_master_resident(qweight.contiguous()), requires_grad=False)
                layer.matgptq_weights = None
            else:
                layer.matgptq_planes = None
                layer.matgptq_weights = Parameter(self._pack_at(layer, qweight, self.bitwidth), requires_grad=False)
            layer.matgptq_bitwidth = self.bitwidth
            layer.matgptq_scales = Parameter(
                torch.ops.matgptq_cuda.reorder_matgptq_scales(
                    layer.scales.data.contiguous(), self.n_out_features, self.n_in_features,
                    self.config.group_size),
                requires_grad=False)
            zeros = getattr(layer, "zeros", None)
            if zeros is not None:
                layer.matgptq_zeros = Parameter(
                    torch.ops.matgptq_cuda.reorder_matgptq_scales(
                        zeros.data.to(layer.scales.dtype).contiguous(), self.n_out_features,
                        self.n_in_features, self.config.group_size),
                    requires_grad=False)
                del layer.zeros
            else:
                layer.matgptq_zeros = None
            perm = getattr(layer, "perm", None)
            if perm is not None:
                # act-order: the codes are stored in permuted column order and the input features
                # are gathered with the permutation (src/quant_utils_matgpqt.py:218-220)
                layer.matgptq_perm = Parameter(perm.data.to(device=layer.matgptq_scales.device,
                                                            dtype=torch.int64).reshape(-1), requires_grad=False)
                del layer.perm
            else:
                layer.matgptq_perm = None

            if self.config.keep_master_codes and not self.config.resident_master_planes:
                # The reference deletes the master codes here (inference_lib/vllm_matgptq.py:177-178);
                # kept, a layer can be re-sliced to another bitwidth without the checkpoint.
                layer.matgptq_master = Parameter(qweight.to(layer.matgptq_scales.device), requires_grad=False)
            del layer.qweight
            del layer.scales

    def set_bitwidth(self, layer: torch.nn.Module, bitwidth: int) -> None:
        """Moves a loaded layer to `bitwidth`.  With `resident_master_planes` nothing is touched but
        the number the next product is called with.  With `keep_master_codes` the layer is re-sliced
        from its resident master codes: one device pass over the codes, not for use inside a captured
        graph (the packed tensor changes size)."""
        if bitwidth not in (2, 3, 4, 6, 8):
            raise ValueError("bitwidth must be one of {2, 3, 4, 6, 8}")
        if getattr(layer, "matgptq_planes", None) is not None:
            layer.matgptq_bitwidth = bitwidth
            return
        master = getattr(layer, "matgptq_master", None)
        if master is None:
            raise RuntimeError("set_bitwidth needs the master codes: load with keep_master_codes "
                               "or resident_master_planes")
        with torch.no_grad():
            layer.matgptq_weights = Parameter(self._pack_at(layer, master.data, bitwidth), requires_grad=False)
            layer.matgptq_bitwidth = bitwidth

    def apply(self, layer: torch.nn.Module, x: torch.Tensor,
              bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        bitwidth = getattr(layer, "matgptq_bitwidth", self.bitwidth)
        if getattr(layer, "matgptq_perm", None) is not None:
            x = torch.index_select(x, -1, layer.matgptq_perm)
        if getattr(layer, "matgptq_planes", None) is not None:
            y = torch.ops.matgptq_cuda.matmul_matgptq_master(
                x, layer.matgptq_planes, layer.matgptq_scales, getattr(layer, "matgptq_zeros", None),
                self.n_out_features, self.n_in_features, bitwidth,
                self.config.group_size, self.config.flag)
        elif getattr(layer, "matgptq_zeros", None) is not None:
            y = torch.ops.matgptq_cuda.matmul_matgptq_zp(
                x, layer.matgptq_weights, layer.matgptq_scales, layer.matgptq_zeros,
                self.n_out_features, self.n_in_features, bitwidth,
                self.config.group_size, self.config.flag)
        else:
            y = torch.ops.matgptq_cuda.matmul_matgptq(
                x, layer.matgptq_weights, layer.matgptq_scales,
                self.n_out_features, self.n_in_features, bitwidth,
                self.config.group_size, self.config.flag)

        y = y.view(*x.shape[:-1], y.shape[-1])
        if bias is not None:
            y += bias
        return y

    def apply_prologue(self, layer: torch.nn.Module, kind: int, a: torch.Tensor, added=None, norm_weight=None,
                       residual_out=None, eps: float = 1e-5) -> torch.Tensor:
        """Additive (no counterpart in the reference): `apply` for decode steps of up to four rows with
        the operator in front of the linear formed inside the kernel - `kind` 1: `a` is the fused
        gate_up output [M, 2K], x = silu(gate) * up; 2: `a` is the residual stream, x = rms_norm(a +
        added) * norm_weight, a + added written to `residual_out`.  Pre-sliced fp16 layers at group
        size 128 without act-order; callers check `matgptq_amd.ops.prologue_applies` first."""
        from matgptq_amd import ops

        if getattr(layer, "matgptq_perm", None) is not None or getattr(layer, "matgptq_planes", None) is not None:
            raise RuntimeError("the fused prologues take pre-sliced layers without an act-order permutation")
        return ops.matmul_matgptq_prologue(kind, a, layer.matgptq_weights, layer.matgptq_scales,
                                           getattr(layer, "matgptq_zeros", None), self.n_out_features,
                                           self.n_in_features, getattr(layer, "matgptq_bitwidth", self.bitwidth),
                                           self.config.group_size, added, norm_weight, residual_out, eps)
