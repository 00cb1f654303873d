"""The torch-op / module / plugin boundary as far as it can be checked without a GPU:
operator names and schemas, fake (meta) shape rules, argument errors, plugin logic."""
import pytest
import torch

import matgptq_cuda
import vllm_matgptq
from matgptq_amd.ops import matryoshka_slice
from matgptq_cuda.matgptq_linear import MatGPTQLinear, MatGTPQ_FeatureFlags

REF_SCHEMAS = {
    # inference_lib/matgptq_cuda/csrc/bindings.cpp:198-200
    "pack_matgptq_qweights": "(Tensor qweights, int n_out_features, int n_in_features, int bitwidth, int group_size, int feature_flag) -> Tensor",
    "reorder_matgptq_scales": "(Tensor scales, int n_out_features, int n_in_features, int group_size) -> Tensor",
    "matmul_matgptq": "(Tensor input, Tensor matgptq_weights, Tensor matgptq_scales, int n_out_features, int n_in_features, int bitwidth, int group_size, int feature_flag) -> Tensor",
}


@pytest.mark.parametrize("ns", ("matgptq_cuda", "_matgptq_cuda_C"))
@pytest.mark.parametrize("name", sorted(REF_SCHEMAS))
def test_reference_schemas(ns, name):
    op = getattr(getattr(torch.ops, ns), name).default
    assert str(op._schema) == f"{ns}::{name}{REF_SCHEMAS[name]}"


def test_python_names_of_the_reference_package():
    for n in REF_SCHEMAS:
        assert callable(getattr(matgptq_cuda, n))
        assert callable(getattr(matgptq_cuda._CUDA, n))
    import matgptq_cuda._CUDA as ext  # the reference's extension-module name

    assert ext.abi_version() == 2
    assert (MatGTPQ_FeatureFlags.SYNC, MatGTPQ_FeatureFlags.ASYNC, MatGTPQ_FeatureFlags.IS_BF16) == (0, 1, 2)
    assert set(["matgptq_qweight", "matgptq_scales"]) <= set(MatGPTQLinear.__init__.__code__.co_names) | {"matgptq_qweight", "matgptq_scales"}


def test_fake_shapes():
    # (input.shape[-2], N), bf16 iff flag bit 1 (inference_lib/matgptq_cuda/__init__.py:49-63)
    with torch.device("meta"):
        w = torch.empty(4 * 32 * 256 // 32, dtype=torch.uint32)
        s = torch.empty(32, 2, dtype=torch.float16)
        x = torch.empty(7, 256, dtype=torch.float16)
        assert torch.ops.matgptq_cuda.matmul_matgptq(x, w, s, 32, 256, 4, 128, 1).shape == (7, 32)
        y = torch.ops.matgptq_cuda.matmul_matgptq(x.view(1, 7, 256), w, s, 32, 256, 4, 128, 3)
        assert y.shape == (7, 32) and y.dtype == torch.bfloat16
        y = torch.ops.matgptq_cuda.matmul_matgptq_zp(x, w, s, s, 32, 256, 4, 128, 1)
        assert y.shape == (7, 32) and y.dtype == torch.float16


def test_argument_errors_match_the_reference_messages():
    q = torch.zeros(16, 128, dtype=torch.uint8)
    pack = torch.ops.matgptq_cuda.pack_matgptq_qweights
    with pytest.raises(RuntimeError, match="qweights must be uint8"):
        pack(q.to(torch.int32), 16, 128, 4, 128, 1)
    with pytest.raises(RuntimeError, match="qweights must be 2D"):
        pack(q.view(-1), 16, 128, 4, 128, 1)
    with pytest.raises(RuntimeError, match="n_out_features does not match"):
        pack(q, 32, 128, 4, 128, 1)
    with pytest.raises(RuntimeError, match=r"bitwidth must be one of \{2, 3, 4, 6, 8\}"):
        pack(q, 16, 128, 5, 128, 1)
    with pytest.raises(RuntimeError, match=r"group_size must be one of \{-1, 32, 128\}"):
        pack(q, 16, 128, 4, 64, 1)
    with pytest.raises(RuntimeError, match="qweights must be contiguous"):
        pack(torch.zeros(128, 16, dtype=torch.uint8).t(), 16, 128, 4, 128, 1)
    with pytest.raises(RuntimeError, match="scales must be contiguous"):
        torch.ops.matgptq_cuda.reorder_matgptq_scales(torch.zeros(16, 4, dtype=torch.float16)[:, ::2], 16, 256, 128)
    with pytest.raises(RuntimeError, match="multiple of 16"):
        pack(torch.zeros(8, 128, dtype=torch.uint8), 8, 128, 4, 128, 1)


@pytest.mark.parametrize("b", (2, 3, 4, 6, 8))
def test_matryoshka_slice_torch_path(b, golden):
    x = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    assert (matryoshka_slice(x, 8, b).numpy() == golden["slice_table"][(2, 3, 4, 6, 8).index(b)]).all()
    with pytest.raises(TypeError):
        matryoshka_slice(x.to(torch.int32), 8, b)


def test_plugin_config_roundtrip():
    cfg = {"group_size": 128, "master_bitwidth": 8, "inference_bitwidth": 3, "quant_dtype": "float16",
           "modules_to_not_convert": ["lm_head", "norm"], "quant_method": "matgptq_quant"}
    c = vllm_matgptq.MatGPTQConfig.from_config(cfg)
    assert (c.group_size, c.master_bitwidth, c.inference_bitwidth, c.quant_dtype) == (128, 8, 3, torch.float16)
    assert c.get_name() == "matgptq_quant" and c.flag == 1 and c.get_config_filenames() == []
    assert c.get_supported_act_dtypes() == [torch.float16, torch.bfloat16]
    assert vllm_matgptq.MatGPTQConfig.get_min_capability() == 80
    with pytest.raises(ValueError):
        vllm_matgptq.MatGPTQConfig.from_config({"group_size": 128})
    with pytest.raises(ValueError):
        vllm_matgptq.MatGPTQConfig(inference_bitwidth=5)


def test_plugin_dispatch_and_per_layer_bits():
    c = vllm_matgptq.MatGPTQConfig(128, 8, 4, "float16", ["lm_head"],
                                   {"layers.0.mlp.down_proj": 2, "down_proj": 6, "qkv_proj": 8})
    lin = vllm_matgptq.LinearBase()
    assert isinstance(c.get_quant_method(lin, "lm_head"), vllm_matgptq.UnquantizedLinearMethod)
    assert c.get_quant_method(torch.nn.ReLU(), "model.act") is None
    assert c.get_quant_method(lin, "model.layers.0.mlp.down_proj").bitwidth == 2   # longest suffix wins
    assert c.get_quant_method(lin, "model.layers.1.mlp.down_proj").bitwidth == 6
    assert c.get_quant_method(lin, "model.layers.1.self_attn.qkv_proj").bitwidth == 8
    assert c.get_quant_method(lin, "model.layers.1.self_attn.o_proj").bitwidth == 4


def test_plugin_create_weights_shapes_and_alignment_error():
    c = vllm_matgptq.MatGPTQConfig(128, 8, 4, "float16", None)
    m = vllm_matgptq.MatGPTQLinearMethod(c)
    layer = torch.nn.Module()
    m.create_weights(layer, 256, [32, 16], 256, 48, torch.float16, weight_loader=None)
    assert layer.qweight.shape == (48, 256) and layer.qweight.dtype == torch.uint8
    assert (layer.qweight.input_dim, layer.qweight.output_dim) == (1, 0)
    assert layer.scales.shape == (48, 2) and layer.scales.dtype == torch.float16
    assert (layer.scales.input_dim, layer.scales.output_dim, layer.scales.packed_dim) == (1, 0, 1)
    with pytest.raises(ValueError, match="not a multiple of the quantisation group size"):
        m.create_weights(torch.nn.Module(), 200, [32], 200, 32, torch.float16)
