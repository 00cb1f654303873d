"""The torch operators, `MatGPTQLinear` and the vLLM quant-method on a real MI355X:
they must give what the C ABI gives (and therefore what the oracle gives)."""
import numpy as np
import pytest
import torch

import matgptq_cuda  # noqa: F401
import vllm_matgptq
from matgptq_amd.ops import matryoshka_slice
from matgptq_cuda.matgptq_linear import MatGPTQLinear
from oracle import matgptq_oracle as o
from tests import _gpu_util as G

pytestmark = pytest.mark.gpu


def _ref(x, q, s, z, b, g):
    return o.dequantize(q, s, z, b, g)


@pytest.mark.parametrize("b", (2, 3, 4, 6, 8))
def test_module_like_the_reference_test(b):
    # construction from host tensors, as inference_lib/test_matgptq_matmul.py:29-47 does
    n, k, g = 64, 1024, 128
    q, s, _ = o.make_layer(n, k, g, seed=b, symmetric=True)
    codes = o.slice_codes(q, b)
    lin = MatGPTQLinear(torch.from_numpy(codes), torch.from_numpy(s), b, g)
    assert lin.matgptq_qweight.dtype == torch.uint32 and lin.matgptq_qweight.is_cuda
    assert lin.matgptq_qweight.numel() == b * n * k // 32
    assert lin.matgptq_scales.shape == (n, k // g) and lin.flag == 1
    w = o.dequantize(q, s, np.full_like(s, 128.0), b, g)
    for m in (1, 8, 33):
        x = o.make_activations(m, k, seed=m)
        y = lin(torch.from_numpy(x).cuda())
        assert y.shape == (m, n) and y.dtype == torch.float16
        G.assert_close_to_oracle(y.cpu().numpy(), x, w, f"module b={b} M={m}")


def test_module_bfloat16():
    # bf16 scales select the bf16 flag (matgptq_linear.py:26 of the reference); output is bf16
    n, k, g, b = 64, 1024, 128, 4
    q, s16, _ = o.make_layer(n, k, g, seed=9, symmetric=True)
    s = o.round_to_bf16(s16.astype(np.float32))
    lin = MatGPTQLinear(torch.from_numpy(o.slice_codes(q, b)), torch.from_numpy(s).to(torch.bfloat16), b, g)
    assert lin.flag == 3 and lin.matgptq_scales.dtype == torch.bfloat16
    w = o.dequantize_bf16(q, s, np.full_like(s, 128.0), b, g)
    for m in (1, 8, 33):
        x = o.round_to_bf16(o.make_activations(m, k, seed=m).astype(np.float32))
        y = lin(torch.from_numpy(x).to(torch.bfloat16).cuda())
        assert y.shape == (m, n) and y.dtype == torch.bfloat16
        ref = o.linear_f64(x, w)
        assert np.max(np.abs(y.float().cpu().numpy() - ref)) <= G.REL_TOL * np.max(np.abs(ref))


def test_ops_accept_device_tensors_and_match_host_packing():
    n, k, b, g = 48, 512, 3, 32
    q, s, z = o.make_layer(n, k, g, seed=2)
    codes = torch.from_numpy(o.slice_codes(q, b))
    p_host = torch.ops.matgptq_cuda.pack_matgptq_qweights(codes, n, k, b, g, 1)
    p_dev = torch.ops.matgptq_cuda.pack_matgptq_qweights(codes.cuda(), n, k, b, g, 1)
    p_master = torch.ops.matgptq_cuda.pack_matgptq_master(torch.from_numpy(q).cuda(), n, k, b, g, 1)
    assert p_host.is_cuda and torch.equal(p_host.cpu().view(torch.int32), p_dev.cpu().view(torch.int32))
    assert torch.equal(p_master.cpu().view(torch.int32), p_dev.cpu().view(torch.int32))
    back = torch.ops.matgptq_cuda.unpack_matgptq_qweights(p_dev, n, k, b)
    assert torch.equal(back.cpu(), codes)
    assert torch.equal(matryoshka_slice(torch.from_numpy(q).cuda(), 8, b).cpu(), codes)
    s_host = torch.ops.matgptq_cuda.reorder_matgptq_scales(torch.from_numpy(s), n, k, g)
    s_dev = torch.ops.matgptq_cuda.reorder_matgptq_scales(torch.from_numpy(s).cuda(), n, k, g)
    assert s_host.is_cuda and s_host.shape == (n, k // g) and torch.equal(s_host, s_dev)
    zr = torch.ops.matgptq_cuda.reorder_matgptq_scales(torch.from_numpy(z).cuda(), n, k, g)
    w = torch.ops.matgptq_cuda.dequantize_matgptq(p_dev, s_dev, zr, n, k, b, g)
    assert np.array_equal(w.cpu().numpy().view(np.uint16), o.dequantize(q, s, z, b, g).view(np.uint16))
    x = o.make_activations(4, k, seed=1)
    y = torch.ops.matgptq_cuda.matmul_matgptq_zp(torch.from_numpy(x).cuda(), p_dev, s_dev, zr, n, k, b, g, 1)
    G.assert_close_to_oracle(y.cpu().numpy(), x, o.dequantize(q, s, z, b, g), "zp op")
    # leading dimensions fold into the batch; a [1, S, K] input gives [S, N] like the reference
    y3 = torch.ops.matgptq_cuda.matmul_matgptq_zp(torch.from_numpy(x).cuda().view(1, 4, k), p_dev, s_dev, zr, n, k, b, g, 1)
    assert torch.equal(y3, y)


def test_op_errors_on_device():
    n, k = 32, 256
    w = torch.zeros(4 * n * k // 32, dtype=torch.uint32, device="cuda")
    s = torch.ones(n, 2, dtype=torch.float16, device="cuda")
    x = torch.ones(1, k, dtype=torch.float16, device="cuda")
    mm = torch.ops.matgptq_cuda.matmul_matgptq
    with pytest.raises(RuntimeError, match="matgptq_weights has the wrong size"):
        mm(x, w[:-1], s, n, k, 4, 128, 1)
    with pytest.raises(RuntimeError, match="matgptq_weights must be uint32"):
        mm(x, w.view(torch.int32), s, n, k, 4, 128, 1)
    with pytest.raises(RuntimeError, match="bitwidth must be one of"):
        mm(x, w, s, n, k, 5, 128, 1)
    with pytest.raises(RuntimeError, match="input must be bfloat16"):
        mm(x, w, s, n, k, 4, 128, 3)  # flag says bf16, tensors are fp16
    with pytest.raises(RuntimeError, match="input must be float16"):
        mm(x.to(torch.bfloat16), w, s.to(torch.bfloat16), n, k, 4, 128, 1)
    with pytest.raises(RuntimeError, match="input must be float16"):
        mm(x.float(), w, s, n, k, 4, 128, 1)
    yb = mm(x.to(torch.bfloat16), w, s.to(torch.bfloat16), n, k, 4, 128, 3)
    assert yb.dtype == torch.bfloat16 and yb.shape == (1, n)
    assert mm(x[:0], w, s, n, k, 4, 128, 1).shape == (0, n)  # empty batch


def test_graph_capture_and_replay():
    # callers wrap the op in graphs (inference_lib/bench_matgptq_matmul.py:48); replays must
    # keep giving the eager result, also with other work between them
    n, k, b, g = 256, 4096, 4, 128
    q, s, z = o.make_layer(n, k, g, seed=5)
    lin = MatGPTQLinear(torch.from_numpy(o.slice_codes(q, b)).cuda(), torch.from_numpy(s).cuda(), b, g,
                        zeros=torch.from_numpy(z).cuda())
    x = torch.from_numpy(o.make_activations(1, k, seed=5)).cuda()
    eager = lin(x).clone()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = lin(x)
    for i in range(4):
        x.copy_(torch.from_numpy(o.make_activations(1, k, seed=5 + i)).cuda())
        expect = lin(x).clone()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, expect)
    x.copy_(torch.from_numpy(o.make_activations(1, k, seed=5)).cuda())
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(y, eager)


@pytest.mark.parametrize("with_zeros", (False, True))
def test_vllm_linear_method_matches_module(with_zeros):
    n1, n2, k, g, b = 64, 32, 512, 128, 3
    q, s, z = o.make_layer(n1 + n2, k, g, seed=9, symmetric=not with_zeros)
    cfg = vllm_matgptq.MatGPTQConfig(g, 8, 4, "float16", ["lm_head"], {"qkv_proj": b})
    layer = vllm_matgptq.LinearBase()
    method = cfg.get_quant_method(layer, "model.layers.0.self_attn.qkv_proj")
    method.create_weights(layer, k, [n1, n2], k, n1 + n2, torch.float16)
    layer.qweight.data.copy_(torch.from_numpy(q))
    layer.scales.data.copy_(torch.from_numpy(s))
    if with_zeros:
        layer.register_parameter("zeros", torch.nn.Parameter(torch.from_numpy(z), requires_grad=False))
    layer.cuda()
    method.process_weights_after_loading(layer)
    assert not hasattr(layer, "qweight") and not hasattr(layer, "scales")
    x = o.make_activations(6, k, seed=3).reshape(2, 3, k)
    bias = torch.arange(n1 + n2, dtype=torch.float16, device="cuda") / 8
    y = method.apply(layer, torch.from_numpy(x).cuda(), bias)
    assert y.shape == (2, 3, n1 + n2)
    w = o.dequantize(q, s, z, b, g)
    got = (y.float() - bias.float()).cpu().numpy().reshape(6, -1)
    ref = o.linear_f64(x.reshape(6, k), w)
    assert np.max(np.abs(got - ref)) <= G.REL_TOL * np.max(np.abs(ref))
    lin = MatGPTQLinear(torch.from_numpy(o.slice_codes(q, b)).cuda(), torch.from_numpy(s).cuda(), b, g,
                        zeros=torch.from_numpy(z).cuda() if with_zeros else None)
    assert torch.equal(lin(torch.from_numpy(x.reshape(6, k)).cuda()) + bias, y.view(6, -1))


@pytest.mark.parametrize("with_zeros", (False, True))
def test_packed_checkpoint_to_module(tmp_path, with_zeros):
    # write a packed checkpoint, read it back, build the modules the transformers demo builds
    # (inference_demo_transformers.py:30-62), compare with the oracle on the stored tensors
    import json
    import os

    from safetensors.torch import save_file

    from matgptq_amd import checkpoint as ck

    model, quant, out = str(tmp_path / "m"), str(tmp_path / "q"), str(tmp_path / "out")
    os.makedirs(model)
    shapes = {"model.layers.0.mlp.up_proj": (64, 512), "model.layers.0.mlp.down_proj": (48, 1024)}
    save_file({f"{k}.weight": torch.zeros(n, kk).half() for k, (n, kk) in shapes.items()},
              os.path.join(model, ck.SINGLE_NAME))
    with open(os.path.join(model, "config.json"), "w") as f:
        json.dump({}, f)
    layers = {}
    for i, (name, (n, k)) in enumerate(shapes.items()):
        q, s, z = o.make_layer(n, k, 128, seed=20 + i, symmetric=not with_zeros)
        data = {"qweight": torch.from_numpy(q), "scale": torch.from_numpy(s)}
        if with_zeros:
            data["zero"] = torch.from_numpy(z)
        os.makedirs(os.path.join(quant, name))
        torch.save(data, os.path.join(quant, name, "data.pt"))
        layers[name] = (q, s, z)
    ck.pack_model(model, quant, out, 128, 8, 4, "float16", layer_bitwidths={"down_proj": 3})
    qc = ck.read_quantization_config(out)
    seen = 0
    for name, tensors in ck.iter_quantised_layers(out):
        bits = ck.bitwidth_of(name, qc)
        assert bits == (3 if name.endswith("down_proj") else 4)
        lin = ck.build_linear(tensors, bits, qc)
        q, s, z = layers[name]
        x = o.make_activations(5, q.shape[1], seed=seen)
        y = lin(torch.from_numpy(x).cuda())
        G.assert_close_to_oracle(y.cpu().numpy(), x, o.dequantize(q, s, z, bits, 128), name)
        seen += 1
    assert seen == 2


def test_mixnmatch_stack_through_plugin():
    # a small Llama-shaped stack whose linears get a bitwidth each from a seeded RNG, configured
    # the way a packed checkpoint's `layer_bitwidths` configures the plugin; every linear is
    # checked against the oracle at its own bitwidth, at batch 1
    import random

    rnd = random.Random(0)
    hidden, ffn, g = 256, 512, 128
    shapes = {"self_attn.qkv_proj": (384, hidden), "self_attn.o_proj": (hidden, hidden),
              "mlp.gate_up_proj": (2 * ffn, hidden), "mlp.down_proj": (hidden, ffn)}
    names = [f"model.layers.{i}.{s}" for i in range(3) for s in shapes]
    bits = {name: rnd.choice((2, 3, 4, 6, 8)) for name in names}
    assert len(set(bits.values())) >= 4
    cfg = vllm_matgptq.MatGPTQConfig.from_config({
        "group_size": g, "master_bitwidth": 8, "inference_bitwidth": 4, "quant_dtype": "float16",
        "modules_to_not_convert": ["lm_head", "norm"], "layer_bitwidths": bits})
    for i, name in enumerate(names):
        n, k = shapes[name.split(".", 3)[3]]
        q, s, _ = o.make_layer(n, k, g, seed=100 + i, symmetric=True)
        layer = vllm_matgptq.LinearBase()
        method = cfg.get_quant_method(layer, name)
        assert method.bitwidth == bits[name]
        method.create_weights(layer, k, [n], k, n, torch.float16)
        layer.qweight.data.copy_(torch.from_numpy(q))
        layer.scales.data.copy_(torch.from_numpy(s))
        layer.cuda()
        method.process_weights_after_loading(layer)
        assert layer.matgptq_weights.numel() == bits[name] * n * k // 32
        x = o.make_activations(1, k, seed=i)
        y = method.apply(layer, torch.from_numpy(x).cuda())
        w = o.dequantize(q, s, np.full_like(s, 128.0), bits[name], g)
        G.assert_close_to_oracle(y.cpu().numpy(), x, w, f"{name} b={bits[name]}")
    assert isinstance(cfg.get_quant_method(vllm_matgptq.LinearBase(), "lm_head"),
                      vllm_matgptq.UnquantizedLinearMethod)
