"""Packed-checkpoint writer/reader: the files carry what the reference's
pack_quantized_model.py writes (tensor names, dtypes, shapes, index, quantization_config keys)."""
import json
import os

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

import vllm_matgptq
from matgptq_amd import checkpoint as ck
from oracle import matgptq_oracle as o

LAYERS = ("model.layers.0.self_attn.q_proj", "model.layers.0.mlp.down_proj")


def _make_model(root, sharded):
    os.makedirs(root)
    tensors = {
        "model.embed_tokens.weight": torch.randn(32, 128).half(),
        "model.layers.0.self_attn.q_proj.weight": torch.randn(32, 128).half(),
        "model.layers.0.mlp.down_proj.weight": torch.randn(16, 256).half(),
        "model.layers.0.input_layernorm.weight": torch.ones(128).half(),
        "model.norm.weight": torch.ones(128).half(),
        "lm_head.weight": torch.randn(32, 128).half(),
    }
    if sharded:
        names = sorted(tensors)
        shards = {"model-00001-of-00002.safetensors": names[:3], "model-00002-of-00002.safetensors": names[3:]}
        wm = {}
        for shard, ns in shards.items():
            save_file({n: tensors[n] for n in ns}, os.path.join(root, shard))
            wm.update({n: shard for n in ns})
        with open(os.path.join(root, ck.INDEX_NAME), "w") as f:
            json.dump({"metadata": {}, "weight_map": wm}, f)
    else:
        save_file(tensors, os.path.join(root, ck.SINGLE_NAME))
    with open(os.path.join(root, "config.json"), "w") as f:
        json.dump({"architectures": ["LlamaForCausalLM"], "hidden_size": 128,
                   "quantization_config": {"quant_method": "something_else"}}, f)
    with open(os.path.join(root, "tokenizer_config.json"), "w") as f:
        json.dump({"model_max_length": 8}, f)
    return tensors


def _make_quantised(root, with_extras):
    os.makedirs(root)
    out = {}
    shapes = {LAYERS[0]: (32, 128), LAYERS[1]: (16, 256), "lm_head": (32, 128)}  # lm_head must be skipped
    for i, (name, (n, k)) in enumerate(shapes.items()):
        q, s, z = o.make_layer(n, k, 128, seed=i)
        data = {"qweight": torch.from_numpy(q), "scale": torch.from_numpy(s).view(n, -1, 1)}
        if with_extras:
            data["zero"] = torch.from_numpy(z).view(n, -1, 1)
            data["perm"] = torch.randperm(k)
        os.makedirs(os.path.join(root, name))
        torch.save(data, os.path.join(root, name, "data.pt"))
        out[name] = data
    open(os.path.join(root, "not_a_layer.txt"), "w").close()
    return out


@pytest.mark.parametrize("sharded", (False, True))
@pytest.mark.parametrize("with_extras", (False, True))
def test_pack_model_writes_the_reference_format(tmp_path, sharded, with_extras):
    model, quant, out = str(tmp_path / "m"), str(tmp_path / "q"), str(tmp_path / "out")
    orig = _make_model(model, sharded)
    qdata = _make_quantised(quant, with_extras)
    wm = ck.pack_model(model, quant, out, 128, 8, 4, "float16",
                       layer_bitwidths={"q_proj": 3} if with_extras else None)

    # every original tensor is there, except the two quantised weights, which became qweight + scales
    got = {}
    for shard in set(wm.values()):
        got.update(load_file(os.path.join(out, shard)))
    assert set(got) == set(wm)
    for name, t in orig.items():
        layer = name.rsplit(".", 1)[0]
        if layer in LAYERS:
            assert name not in got
            assert got[f"{layer}.qweight"].dtype == torch.uint8
            assert torch.equal(got[f"{layer}.qweight"], qdata[layer]["qweight"])
            n = t.shape[0]
            assert got[f"{layer}.scales"].shape == (n, t.shape[1] // 128)
            assert torch.equal(got[f"{layer}.scales"], qdata[layer]["scale"].view(n, -1))
            assert (f"{layer}.zeros" in got) == with_extras and (f"{layer}.perm" in got) == with_extras
            if with_extras:
                assert torch.equal(got[f"{layer}.zeros"], qdata[layer]["zero"].view(n, -1))
                assert torch.equal(got[f"{layer}.perm"].long(), qdata[layer]["perm"])
        else:
            assert torch.equal(got[name], t)  # lm_head and norms stay dense
    # a quantised tensor lives in the shard its weight came from
    if sharded:
        with open(os.path.join(model, ck.INDEX_NAME)) as f:
            old = json.load(f)["weight_map"]
        with open(os.path.join(out, ck.INDEX_NAME)) as f:
            new = json.load(f)
        assert new["metadata"] == {} and new["weight_map"] == wm
        for layer in LAYERS:
            assert wm[f"{layer}.qweight"] == wm[f"{layer}.scales"] == old[f"{layer}.weight"]
    else:
        assert set(wm.values()) == {ck.SINGLE_NAME}

    # config: previous quantization_config replaced, keys of pack_quantized_model.py:134-141
    with open(os.path.join(out, "config.json")) as f:
        cfg = json.load(f)
    qc = cfg["quantization_config"]
    assert cfg["hidden_size"] == 128
    assert {k: qc[k] for k in ("group_size", "modules_to_not_convert", "master_bitwidth", "inference_bitwidth",
                               "quant_method", "quant_dtype")} == {
        "group_size": 128, "modules_to_not_convert": ["lm_head", "norm"], "master_bitwidth": 8,
        "inference_bitwidth": 4, "quant_method": "matgptq_quant", "quant_dtype": "float16"}
    assert os.path.exists(os.path.join(out, "tokenizer_config.json"))
    # the vLLM plugin accepts it
    c = vllm_matgptq.MatGPTQConfig.from_config(qc)
    assert c.inference_bitwidth == 4 and c.group_size == 128
    assert c.bitwidth_for(LAYERS[0]) == (3 if with_extras else 4)
    # zeros / perm are announced in the config exactly when the shards carry them
    assert qc.get("has_zeros", False) == with_extras and qc.get("has_perm", False) == with_extras
    assert c.has_zeros == with_extras and c.has_perm == with_extras

    # reader
    assert ck.read_quantization_config(out) == qc
    layers = dict(ck.iter_quantised_layers(out))
    assert set(layers) == set(LAYERS)
    assert ck.bitwidth_of(LAYERS[0], qc) == (3 if with_extras else 4) and ck.bitwidth_of(LAYERS[1], qc) == 4
    for layer, t in layers.items():
        assert torch.equal(t["qweight"], qdata[layer]["qweight"])
        assert ("zeros" in t) == with_extras


def test_pack_model_errors(tmp_path):
    model, quant = str(tmp_path / "m"), str(tmp_path / "q")
    _make_model(model, False)
    _make_quantised(quant, False)
    with pytest.raises(ValueError, match="quant_dtype"):
        ck.pack_model(model, quant, str(tmp_path / "o1"), 128, 8, 4, "float32")
    with pytest.raises(ValueError, match="scale has"):
        ck.pack_model(model, quant, str(tmp_path / "o2"), 32, 8, 4, "float16")
    os.remove(os.path.join(quant, LAYERS[0], "data.pt"))
    with pytest.raises(FileNotFoundError, match="No data.pt"):
        ck.pack_model(model, quant, str(tmp_path / "o3"), 128, 8, 4, "float16")
    os.remove(os.path.join(model, ck.SINGLE_NAME))
    with pytest.raises(FileNotFoundError, match="Neither"):
        ck.pack_model(model, quant, str(tmp_path / "o4"), 128, 8, 4, "float16")
    with pytest.raises(ValueError, match="no matgptq_quant"):
        ck.read_quantization_config(model)


def test_layer_bitwidth_file(tmp_path):
    p = tmp_path / "bits.txt"
    p.write_text("model.layers.0.self_attn.q_proj: 3\n\nmodel.layers.0.mlp.down_proj:6\n")
    assert ck.read_layer_bitwidths(str(p)) == {LAYERS[0]: 3, LAYERS[1]: 6}
    assert np.all([not ck.should_skip_quantisation(x) for x in LAYERS])
    assert ck.should_skip_quantisation("lm_head") and ck.should_skip_quantisation("model.norm")


def test_symmetric_zeros_and_identity_perm_are_not_written(tmp_path):
    # the reference quantiser always stores a `zero` (128 everywhere for symmetric recipes) and its
    # plugin registers only qweight and scales: such a checkpoint must not carry tensors a loader
    # has no parameter for
    model, quant, out = str(tmp_path / "m"), str(tmp_path / "q"), str(tmp_path / "out")
    _make_model(model, False)
    os.makedirs(quant)
    for i, (name, (n, k)) in enumerate({LAYERS[0]: (32, 128), LAYERS[1]: (16, 256)}.items()):
        q, s, _ = o.make_layer(n, k, 128, seed=i)
        os.makedirs(os.path.join(quant, name))
        torch.save({"qweight": torch.from_numpy(q), "scale": torch.from_numpy(s),
                    "zero": torch.full((n, k // 128), 128.0).half(), "perm": torch.arange(k)},
                   os.path.join(quant, name, "data.pt"))
    wm = ck.pack_model(model, quant, out, 128, 8, 4, "float16")
    assert not any(name.endswith((".zeros", ".perm")) for name in wm)
    qc = ck.read_quantization_config(out)
    assert "has_zeros" not in qc and "has_perm" not in qc


def test_mixed_layers_get_zeros_everywhere(tmp_path):
    # one asymmetric layer makes the checkpoint asymmetric: every quantised linear then carries
    # zeros (128 where the quantiser stored none), because the plugin registers them per config
    model, quant, out = str(tmp_path / "m"), str(tmp_path / "q"), str(tmp_path / "out")
    _make_model(model, False)
    os.makedirs(quant)
    q0, s0, z0 = o.make_layer(32, 128, 128, seed=0)
    q1, s1, _ = o.make_layer(16, 256, 128, seed=1)
    for name, data in ((LAYERS[0], {"qweight": q0, "scale": s0, "zero": z0}), (LAYERS[1], {"qweight": q1, "scale": s1})):
        os.makedirs(os.path.join(quant, name))
        torch.save({k: torch.from_numpy(v) for k, v in data.items()}, os.path.join(quant, name, "data.pt"))
    wm = ck.pack_model(model, quant, out, 128, 8, 4, "float16")
    got = load_file(os.path.join(out, ck.SINGLE_NAME))
    assert torch.equal(got[f"{LAYERS[0]}.zeros"], torch.from_numpy(z0))
    assert torch.equal(got[f"{LAYERS[1]}.zeros"], torch.full((16, 2), 128.0).half())
    assert ck.read_quantization_config(out)["has_zeros"] is True and f"{LAYERS[1]}.perm" not in wm


def _strict_load(layer: torch.nn.Module, tensors: dict) -> None:
    """What a model loader does with a layer's tensors: every name must have a registered
    parameter of the same shape and dtype; unknown names are an error."""
    params = dict(layer.named_parameters())
    for name, t in tensors.items():
        if name not in params:
            raise KeyError(f"unexpected tensor {name}")
        assert params[name].shape == t.shape and params[name].dtype == t.dtype, name
        params[name].data.copy_(t)


@pytest.mark.parametrize("with_extras", (False, True))
def test_plugin_registers_what_the_checkpoint_carries(tmp_path, with_extras):
    model, quant, out = str(tmp_path / "m"), str(tmp_path / "q"), str(tmp_path / "out")
    _make_model(model, False)
    _make_quantised(quant, with_extras)
    ck.pack_model(model, quant, out, 128, 8, 4, "float16")
    qc = ck.read_quantization_config(out)
    config = vllm_matgptq.MatGPTQConfig.from_config(qc)
    for name, tensors in ck.iter_quantised_layers(out):
        n, k = tensors["qweight"].shape
        layer = torch.nn.Module()
        method = vllm_matgptq.MatGPTQLinearMethod(config, config.bitwidth_for(name))
        method.create_weights(layer, k, [n], k, n, torch.float16)
        assert set(dict(layer.named_parameters())) == set(tensors)
        _strict_load(layer, tensors)
    # a config without the flags registers neither, and the same tensors are then refused
    plain = vllm_matgptq.MatGPTQConfig.from_config({k: v for k, v in qc.items() if k not in ("has_zeros", "has_perm")})
    layer = torch.nn.Module()
    vllm_matgptq.MatGPTQLinearMethod(plain).create_weights(layer, 128, [32], 128, 32, torch.float16)
    assert set(dict(layer.named_parameters())) == {"qweight", "scales"}
    if with_extras:
        with pytest.raises(KeyError, match="unexpected tensor"):
            _strict_load(layer, dict(ck.iter_quantised_layers(out))[LAYERS[0]])
        # act-order and a split of in_features do not go together
        with pytest.raises(ValueError, match="act-order"):
            vllm_matgptq.MatGPTQLinearMethod(config).create_weights(torch.nn.Module(), 128, [32], 256, 32, torch.float16)
