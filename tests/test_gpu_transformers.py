"""The reference's transformers caller on a real `LlamaForCausalLM`
(inference_lib/inference_demo_transformers.py:17-56 `replace_with_matgptq_linear`, :132-175 decode
with `StaticCache` under `torch.compile(fullgraph=True, mode="reduce-overhead")`;
bench_transformers_e2e.py:61-76 `time_prof`).

The model is built from a local `LlamaConfig` with random weights (nothing is fetched); every
linear of every block is replaced by a `MatGPTQLinear` read from per-layer `data.pt` files at a
seeded per-layer bitwidth, and compared with the same model holding the oracle's dequantised
weights in plain `nn.Linear` modules.
"""
import os
import random

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

transformers = pytest.importorskip("transformers")

from oracle import matgptq_oracle as o  # noqa: E402

LINEARS = ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "self_attn.o_proj",
           "mlp.gate_proj", "mlp.up_proj", "mlp.down_proj")
GROUP = 128


def _tiny_llama(seed=0):
    from transformers import LlamaConfig, LlamaForCausalLM

    cfg = LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                      num_key_value_heads=2, vocab_size=512, max_position_embeddings=256, rms_norm_eps=1e-5,
                      rope_theta=10000.0, tie_word_embeddings=False, attention_bias=False, mlp_bias=False)
    torch.manual_seed(seed)
    model = LlamaForCausalLM(cfg).to(torch.float16).eval()
    return cfg, model


def _write_quantised_layers(model, root, symmetric):
    """Seeded master codes, scales (and zeros) for every block linear as the quantiser's per-layer
    directories; returns `name -> (q, s, z)`.  Scales are sized so that the residual stream of the
    random model stays well inside fp16."""
    layers = {}
    idx = 0
    for li in range(model.config.num_hidden_layers):
        for short in LINEARS:
            name = f"model.layers.{li}.{short}"
            lin = model.get_submodule(name)
            n, k = lin.weight.shape
            q, s, z = o.make_layer(n, k, GROUP, seed=100 + idx, symmetric=symmetric)
            s = (s.astype(np.float32) * 0.04).astype(np.float16)
            os.makedirs(os.path.join(root, name))
            data = {"qweight": torch.from_numpy(q), "scale": torch.from_numpy(s)}
            if not symmetric:
                data["zero"] = torch.from_numpy(z)
            torch.save(data, os.path.join(root, name, "data.pt"))
            layers[name] = (q, s, z)
            idx += 1
    return layers


def _bits_file(layers, path, seed=0):
    rnd = random.Random(seed)
    bits = {name: rnd.choice((2, 3, 4, 6, 8)) for name in layers}
    with open(path, "w") as f:
        for name, b in bits.items():
            f.write(f"{name}: {b}\n")
    return bits


def _pair(tmp_path, symmetric=True):
    """(model with MatGPTQLinear modules, model with the oracle's dense weights, bits)."""
    from matgptq_amd.decoder import replace_with_matgptq_linear
    from matgptq_cuda.matgptq_linear import MatGPTQLinear

    _, quant = _tiny_llama()
    _, dense = _tiny_llama()
    layers = _write_quantised_layers(quant, str(tmp_path), symmetric)
    bits = _bits_file(layers, str(tmp_path / "bits.txt"))
    quant = quant.cuda()
    replace_with_matgptq_linear(quant, str(tmp_path), str(tmp_path / "bits.txt"), master_bitwidth=8,
                                slice_bitwidth=8, group_size=GROUP)
    for name, (q, s, z) in layers.items():
        mod = quant.get_submodule(name)
        assert isinstance(mod, MatGPTQLinear) and mod.bitwidth == bits[name]
        w = o.dequantize(q, s, z, bits[name], GROUP)
        dense.get_submodule(name).weight.data = torch.from_numpy(w)
    assert isinstance(quant.lm_head, torch.nn.Linear)
    return quant, dense.cuda(), bits


@pytest.mark.parametrize("symmetric", (True, False))
def test_logits_match_the_model_with_the_oracles_dense_weights(tmp_path, symmetric):
    quant, dense, bits = _pair(tmp_path, symmetric)
    assert len(set(bits.values())) >= 3  # a real Mix'n'Match assignment
    ids = torch.randint(0, 512, (1, 24), generator=torch.Generator().manual_seed(1)).cuda()
    with torch.no_grad():
        a = quant(ids, use_cache=False).logits.float()
        b = dense(ids, use_cache=False).logits.float()
        one = quant(ids[:, :1], use_cache=False).logits.float()  # a single row: the gemv kernel
        one_ref = dense(ids[:, :1], use_cache=False).logits.float()
    assert torch.isfinite(a).all()
    assert (a - b).abs().max().item() <= 1e-2 * b.abs().max().item()
    assert (one - one_ref).abs().max().item() <= 1e-2 * one_ref.abs().max().item()


def _decode_one_tokens(model, cur_token, input_pos, cache_position, past_key_values):
    logits = model(cur_token, position_ids=input_pos, cache_position=cache_position,
                   past_key_values=past_key_values, return_dict=False, use_cache=True)[0]
    return torch.argmax(logits[:, -1], dim=-1)[:, None]


def _generate(model, ids, new_tokens, decode_fn):
    from transformers import StaticCache

    seq_len = ids.shape[1]
    cache = StaticCache(config=model.config, max_batch_size=1, max_cache_len=seq_len + new_tokens,
                        device=ids.device, dtype=torch.float16)
    cache_position = torch.arange(seq_len, dtype=torch.int64, device=ids.device)
    out = []
    with torch.no_grad():
        logits = model(ids, cache_position=cache_position, past_key_values=cache, return_dict=False,
                       use_cache=True)[0]
        next_token = torch.argmax(logits[:, [-1]], dim=-1)
        out.append(next_token.clone())
        cache_position = torch.tensor([seq_len], device=ids.device)
        for _ in range(1, new_tokens):
            next_token = decode_fn(model, next_token.clone(), None, cache_position, cache)
            out.append(next_token.clone())
            cache_position += 1
    return torch.cat(out, dim=1)


def test_greedy_decode_with_static_cache_compiled_equals_eager(tmp_path):
    quant, dense, _ = _pair(tmp_path)
    ids = torch.randint(0, 512, (1, 9), generator=torch.Generator().manual_seed(2)).cuda()
    eager = _generate(quant, ids, 12, _decode_one_tokens)
    torch._dynamo.config.capture_scalar_outputs = True
    try:
        fn = torch.compile(_decode_one_tokens, fullgraph=True, dynamic=True, mode="reduce-overhead")
        compiled = _generate(quant, ids, 12, fn)
        print("transformers decode: inductor ran")
    except Exception as e:  # the inductor toolchain may be absent; graph breaks are failures
        if "fullgraph" in str(e).lower() or "graph break" in str(e).lower():
            raise
        print(f"transformers decode: inductor unavailable ({type(e).__name__}: {str(e)[:200]}), aot_eager instead")
        torch._dynamo.reset()
        fn = torch.compile(_decode_one_tokens, fullgraph=True, dynamic=True, backend="aot_eager")
        compiled = _generate(quant, ids, 12, fn)
    assert torch.equal(eager, compiled), (eager, compiled)
    # the first token comes from the prompt's logits, which the test above holds to the oracle's
    ref = _generate(dense, ids, 1, _decode_one_tokens)
    assert torch.equal(eager[:, :1], ref)
