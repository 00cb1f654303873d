"""The callers of the linear: module replacement from layer directories and the decoder with
a static cache whose step is captured into a graph (counterparts of
inference_lib/inference_demo_transformers.py:17-56,134-176)."""
import os

import numpy as np
import pytest
import torch

from oracle import matgptq_oracle as o

pytestmark = pytest.mark.gpu

TINY = dict(hidden=256, ffn=512, layers=2, heads=4, kv_heads=2, vocab=512)


class _Dense(torch.nn.Module):
    def __init__(self, w: np.ndarray):
        super().__init__()
        self.w = torch.from_numpy(w.astype(np.float32)).cuda()

    def forward(self, x):
        return (x.float() @ self.w.T).to(x.dtype)


def _tiny(bit_choices=(2, 3, 4, 6, 8), seed=3, context=96):
    from matgptq_amd import decoder as D

    cfg = D.DecoderConfig(**TINY)
    dec, bits, masters = D.random_mixnmatch_decoder(cfg, context, bit_choices, seed=seed, keep_master=True)
    return D, cfg, dec, bits, masters


def test_decoder_matches_dense_decoder_on_oracle_weights():
    D, cfg, dec, bits, masters = _tiny()
    assert sorted(set(bits.values())) != [4]  # several bitwidths in one model
    blocks = []
    for i in range(cfg.layers):
        lin = {}
        for name in cfg.linear_shapes():
            codes, scale, zero = masters[f"blocks.{i}.{name}"]
            w = o.dequantize(codes.cpu().numpy(), scale.cpu().numpy(), zero.cpu().numpy(),
                             bits[f"blocks.{i}.{name}"], cfg.group_size)
            lin[name] = _Dense(w)
        blocks.append(D.Block(cfg, lin, torch.float16, "cuda"))
    ref = D.Decoder(cfg, blocks, dec.embed.data, dec.head.data, dec.max_context)
    prompt = torch.randint(0, cfg.vocab, (40,), device="cuda", generator=torch.Generator(device="cuda").manual_seed(1))
    pos = torch.arange(40, device="cuda")
    a = dec(prompt, pos, dec.new_cache())
    b = ref(prompt, pos, ref.new_cache())
    # two fp16 pipelines over 2 blocks: tolerance 2e-2 of the largest logit
    assert float((a - b).abs().max()) <= 2e-2 * float(b.abs().max())
    # decode kernels (M = 1) continue what the prefill kernels (M = 40) started
    s = D.DecodeSession(dec)
    s.prefill(prompt[:39])
    s.token.copy_(prompt[39:40])
    s.step()
    assert float((s.logits - b).abs().max()) <= 2e-2 * float(b.abs().max())


def test_graph_replays_equal_eager_steps():
    D, cfg, dec, bits, _ = _tiny(seed=5)
    prompt = torch.randint(0, cfg.vocab, (32,), device="cuda", generator=torch.Generator(device="cuda").manual_seed(2))
    eager = D.DecodeSession(dec)
    eager.prefill(prompt)
    graphed = D.DecodeSession(dec)
    graphed.prefill(prompt)
    graphed.capture()
    assert torch.equal(eager.token, graphed.token) and torch.equal(eager.pos, graphed.pos)
    assert torch.equal(eager.cache, graphed.cache)  # the capture left no trace
    for i in range(12):
        eager.step()
        graphed.replay()
        torch.cuda.synchronize()
        # eager work and synchronisation between replays; every replay is checked
        assert torch.equal(eager.logits, graphed.logits), f"replay {i}"
        assert torch.equal(eager.token, graphed.token), f"replay {i}"
        assert int(graphed.pos.item()) == 33 + i
    assert torch.equal(eager.cache, graphed.cache)
    out = D.DecodeSession(dec).generate(prompt, 13, use_graph=True)
    out_eager = D.DecodeSession(dec).generate(prompt, 13, use_graph=False)
    assert torch.equal(out, out_eager)


def test_plugin_built_decoder_equals_module_built_decoder():
    from matgptq_amd import decoder as D

    cfg = D.DecoderConfig(**TINY)
    a, bits_a, _ = D.random_mixnmatch_decoder(cfg, 64, seed=9)
    b, bits_b, _ = D.random_mixnmatch_decoder(cfg, 64, seed=9, via_plugin=True)
    assert bits_a == bits_b and len(set(bits_a.values())) >= 3
    assert all(isinstance(blk.qkv, D.PluginLinear) for blk in b.blocks)
    prompt = torch.randint(0, cfg.vocab, (20,), device="cuda", generator=torch.Generator(device="cuda").manual_seed(4))
    ta = D.DecodeSession(a).generate(prompt, 6, use_graph=True)
    tb = D.DecodeSession(b).generate(prompt, 6, use_graph=True)
    assert torch.equal(ta, tb)
    pos = torch.arange(20, device="cuda")
    assert torch.equal(a(prompt, pos, a.new_cache()), b(prompt, pos, b.new_cache()))


def test_cache_limits_raise():
    D, cfg, dec, _, _ = _tiny(bit_choices=(4,), context=48)
    s = D.DecodeSession(dec)
    with pytest.raises(ValueError):
        s.generate(torch.zeros(40, dtype=torch.int64, device="cuda"), 16)
    with pytest.raises(ValueError):
        s.prefill(torch.zeros(48, dtype=torch.int64, device="cuda"))


@pytest.mark.parametrize("per_layer_file", [False, True])
def test_replace_with_matgptq_linear(tmp_path, per_layer_file):
    from matgptq_amd.decoder import replace_with_matgptq_linear
    from matgptq_cuda.matgptq_linear import MatGPTQLinear

    class Mlp(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.up_proj = torch.nn.Linear(256, 64, bias=False)
            self.down_proj = torch.nn.Linear(128, 48, bias=False)

    class Model(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.layers = torch.nn.ModuleList([Mlp()])
            self.lm_head = torch.nn.Linear(256, 32, bias=False)

    model = Model()
    layers = {}
    for i, (name, (n, k)) in enumerate({"layers.0.up_proj": (64, 256), "layers.0.down_proj": (48, 128)}.items()):
        q, s, z = o.make_layer(n, k, 128, seed=40 + i, symmetric=(i == 0))
        data = {"qweight": torch.from_numpy(q), "scale": torch.from_numpy(s)}
        if i == 1:
            data["zero"] = torch.from_numpy(z)
        os.makedirs(tmp_path / name)
        torch.save(data, tmp_path / name / "data.pt")
        layers[name] = (q, s, z)
    cfg_path = None
    want = {"layers.0.up_proj": 6, "layers.0.down_proj": 6}
    if per_layer_file:
        cfg_path = str(tmp_path / "bits.txt")
        with open(cfg_path, "w") as f:
            f.write("layers.0.up_proj: 3\nlayers.0.down_proj: 8\n")
        want = {"layers.0.up_proj": 3, "layers.0.down_proj": 8}
    replace_with_matgptq_linear(model, str(tmp_path), cfg_path, master_bitwidth=8, slice_bitwidth=6, group_size=128)
    assert isinstance(model.lm_head, torch.nn.Linear)
    from tests import _gpu_util as G
    for name, (q, s, z) in layers.items():
        mod = model.get_submodule(name)
        assert isinstance(mod, MatGPTQLinear) and mod.bitwidth == want[name]
        x = o.make_activations(3, q.shape[1], seed=7)
        y = mod(torch.from_numpy(x).cuda())
        G.assert_close_to_oracle(y.cpu().numpy(), x, o.dequantize(q, s, z, want[name], 128), name)
