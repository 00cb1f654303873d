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


def test_act_order_permutation_is_applied():
    # FakeMatryoshkaLinear.forward gathers the input features with `perm` before the product
    # (src/quant_utils_matgpqt.py:218-220): the codes are stored in permuted column order
    n, k, g, b = 64, 1024, 128, 4
    q, s, z = o.make_layer(n, k, g, seed=31)
    perm = np.random.default_rng(3).permutation(k)
    w = o.dequantize(q, s, z, b, g)
    lin = MatGPTQLinear(torch.from_numpy(o.slice_codes(q, b)), torch.from_numpy(s), b, g,
                        zeros=torch.from_numpy(z), perm=torch.from_numpy(perm))
    plain = MatGPTQLinear(torch.from_numpy(o.slice_codes(q, b)), torch.from_numpy(s), b, g, zeros=torch.from_numpy(z))
    for m in (1, 3, 40):
        x = o.make_activations(m, k, seed=m)
        y = lin(torch.from_numpy(x).cuda()).cpu().numpy()
        G.assert_close_to_oracle(y, x[:, perm], w, f"perm M={m}")
        # equivalently: the dense weight with its columns put back (src/model_utils.py:185-195)
        G.assert_close_to_oracle(y, x, w[:, np.argsort(perm)], f"perm, dense form M={m}")
        assert not np.allclose(y, plain(torch.from_numpy(x).cuda()).cpu().numpy(), rtol=1e-2, atol=1e-2)
    with pytest.raises(ValueError, match="n_in_features"):
        MatGPTQLinear(torch.from_numpy(o.slice_codes(q, b)), torch.from_numpy(s), b, g, perm=torch.arange(k - 1))


def test_plugin_loads_an_act_order_asymmetric_checkpoint(tmp_path):
    # packed checkpoint with zeros and perm -> create_weights -> a loader that refuses unknown
    # names -> process_weights_after_loading -> apply, against the oracle; build_linear agrees
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
    rng = np.random.default_rng(1)
    for i, (name, (n, k)) in enumerate(shapes.items()):
        q, s, z = o.make_layer(n, k, 128, seed=50 + i)
        perm = rng.permutation(k)
        os.makedirs(os.path.join(quant, name))
        torch.save({"qweight": torch.from_numpy(q), "scale": torch.from_numpy(s), "zero": torch.from_numpy(z),
                    "perm": torch.from_numpy(perm)}, os.path.join(quant, name, "data.pt"))
        layers[name] = (q, s, z, perm)
    ck.pack_model(model, quant, out, 128, 8, 4, "float16", layer_bitwidths={"down_proj": 3})
    qc = ck.read_quantization_config(out)
    assert qc["has_zeros"] and qc["has_perm"]
    config = vllm_matgptq.MatGPTQConfig.from_config(qc)
    for name, tensors in ck.iter_quantised_layers(out):
        q, s, z, perm = layers[name]
        n, k = q.shape
        bits = config.bitwidth_for(name)
        layer = torch.nn.Module()
        method = vllm_matgptq.MatGPTQLinearMethod(config, bits)
        method.create_weights(layer, k, [n], k, n, torch.float16)
        layer.cuda()
        params = dict(layer.named_parameters())
        for key, t in tensors.items():
            assert key in params, f"the loader has no destination for {key}"
            params[key].data.copy_(t)
        method.process_weights_after_loading(layer)
        assert not hasattr(layer, "qweight") and not hasattr(layer, "perm") and not hasattr(layer, "zeros")
        w = o.dequantize(q, s, z, bits, 128)
        x = o.make_activations(5, k, seed=bits)
        y = method.apply(layer, torch.from_numpy(x).cuda())
        G.assert_close_to_oracle(y.cpu().numpy(), x[:, perm], w, name)
        y2 = ck.build_linear(tensors, bits, qc)(torch.from_numpy(x).cuda())
        assert torch.equal(y, y2)


def test_resident_master_codes_switch_bitwidth_at_run_time():
    # the reference deletes the master codes after loading (inference_lib/vllm_matgptq.py:177-178);
    # kept resident, a layer moves between bitwidths without the checkpoint
    n, k = 96, 1024
    q, s, z = o.make_layer(n, k, 128, seed=77)
    config = vllm_matgptq.MatGPTQConfig(128, 8, 4, "float16", None, keep_master_codes=True)
    layer = torch.nn.Module()
    method = vllm_matgptq.MatGPTQLinearMethod(config)
    method.create_weights(layer, k, [n], k, n, torch.float16)
    layer.cuda()
    layer.qweight.data.copy_(torch.from_numpy(q))
    layer.scales.data.copy_(torch.from_numpy(s))
    layer.zeros = torch.nn.Parameter(torch.from_numpy(z).cuda(), requires_grad=False)
    method.process_weights_after_loading(layer)
    assert torch.equal(layer.matgptq_master.cpu(), torch.from_numpy(q))
    x = o.make_activations(3, k, seed=5)
    xd = torch.from_numpy(x).cuda()
    for bits in (4, 2, 8, 3, 6, 4):
        method.set_bitwidth(layer, bits)
        assert layer.matgptq_weights.numel() == bits * n * k // 32
        G.assert_close_to_oracle(method.apply(layer, xd).cpu().numpy(), x, o.dequantize(q, s, z, bits, 128), f"b={bits}")
        codes = torch.ops.matgptq_cuda.unpack_matgptq_qweights(layer.matgptq_weights, n, k, bits)
        assert np.array_equal(codes.cpu().numpy(), o.slice_codes(q, bits))
    with pytest.raises(ValueError):
        method.set_bitwidth(layer, 5)
    plain = vllm_matgptq.MatGPTQLinearMethod(vllm_matgptq.MatGPTQConfig(128, 8, 4, "float16", None))
    with pytest.raises(RuntimeError, match="keep_master_codes"):
        plain.set_bitwidth(torch.nn.Module(), 4)


def test_strided_input_is_accepted():
    # the reference never checks the layout of its input (bindings.cpp:146-191)
    n, k, b = 64, 512, 4
    q, s, z = o.make_layer(n, k, 128, seed=8)
    lin = MatGPTQLinear(torch.from_numpy(o.slice_codes(q, b)), torch.from_numpy(s), b, 128, zeros=torch.from_numpy(z))
    x = o.make_activations(6, 2 * k, seed=1)
    xd = torch.from_numpy(x).cuda()
    y = lin(xd[:, :k])  # a slice of a wider tensor: row stride 2k
    G.assert_close_to_oracle(y.cpu().numpy(), x[:, :k], o.dequantize(q, s, z, b, 128), "strided input")


@pytest.mark.parametrize("mode", ("default", "reduce-overhead"))
def test_torch_compile_fullgraph(mode):
    # how the reference's callers run decode (inference_lib/inference_demo_transformers.py:161-162,
    # bench_matgptq_matmul.py:48): torch.compile(fullgraph=True) over modules that contain the
    # operator, which needs nothing but its fake implementation
    n, k, b = 256, 1024, 4
    q, s, z = o.make_layer(n, k, 128, seed=4)

    class Mlp(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.up = MatGPTQLinear(torch.from_numpy(o.slice_codes(q, b)), torch.from_numpy(s), b, 128,
                                    zeros=torch.from_numpy(z))
            self.sym = MatGPTQLinear(torch.from_numpy(o.slice_codes(q[:, :256].copy(), 3)), torch.from_numpy(s[:, :2].copy()), 3, 128)

        def forward(self, x):
            h = torch.nn.functional.silu(self.up(x))
            return h + self.sym(h)

    mod = Mlp().cuda()
    x = torch.from_numpy(o.make_activations(1, k, seed=2)).cuda()
    eager = mod(x)
    try:
        compiled = torch.compile(mod, fullgraph=True, mode=mode)
        got = [compiled(x).clone() for _ in range(4)]  # warm-up, capture and replays
        print(f"torch.compile mode={mode}: inductor ran")
    except Exception as e:  # the inductor toolchain (a C++ compiler for its wrapper) may be absent
        if "fullgraph" in str(e).lower() or "graph break" in str(e).lower():
            raise
        print(f"torch.compile mode={mode}: inductor unavailable ({type(e).__name__}), aot_eager instead")
        compiled = torch.compile(mod, fullgraph=True, backend="aot_eager")
        got = [compiled(x).clone() for _ in range(2)]
    torch.cuda.synchronize()
    for g in got:
        assert torch.allclose(g, eager, rtol=1e-3, atol=1e-3)
    G.assert_close_to_oracle(mod.up(x).cpu().numpy(), x.cpu().numpy(), o.dequantize(q, s, z, b, 128), "compiled module's linear")
