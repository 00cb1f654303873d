"""The benchmark configurations at their stated shapes, through the planner's default choice,
against the oracle (the smaller parity tests cover every kernel variant on small layers)."""
import numpy as np
import pytest
import torch

from matgptq_amd import _lib
from oracle import matgptq_oracle as o
from tests import _gpu_util as G

pytestmark = pytest.mark.gpu

LLAMA8B = {"qkv": (6144, 4096), "o": (4096, 4096), "gate_up": (28672, 4096), "down": (4096, 14336)}
LLAMA70B = {"qkv": (10240, 8192), "o": (8192, 8192), "gate_up": (57344, 8192), "down": (8192, 28672)}

# kernel the planner takes per layer and batch size (eight batch rows: the gemv kernel up to 512 row
# blocks; 4 and 3 bits take the same, except that 3 bits
# take four row blocks per workgroup on the layer with many rows at four batch rows: `{r}`)
SMALL_BATCH_PLANS = {
    "qkv": {2: "gemv b{b} g128 zp1 T4 R1 W8 pad0", 4: "gemv b{b} g128 zp1 T4 R2 W8 pad0",
            8: "gemv b{b} g128 zp1 T4 R2 W8 pad0", 16: "midbatch b{b} g128 zp1 R2 mb1"},
    "o": {2: "gemv b{b} g128 zp1 T4 R1 W8 pad0", 4: "gemv b{b} g128 zp1 T4 R1 W8 pad0",
          8: "gemv b{b} g128 zp1 T4 R1 W8 pad0", 16: "midbatch b{b} g128 zp1 R1 mb1"},
    "gate_up": {2: "gemv b{b} g128 zp1 T4 R1 W8 pad0", 4: "gemv b{b} g128 zp1 T4 R{r} W8 pad0",
                8: "midbatch b{b} g128 zp1 R4 mb1", 16: "midbatch b{b} g128 zp1 R4 mb1"},
    "down": {2: "gemv b{b} g128 zp1 T4 R1 W16 pad0", 4: "gemv b{b} g128 zp1 T4 R1 W16 pad0",
             8: "gemv b{b} g128 zp1 T4 R1 W16 pad0", 16: "midbatch b{b} g128 zp1 R1 mb1"},
}


@pytest.mark.parametrize("name", sorted(LLAMA8B))
@pytest.mark.parametrize("b", (3, 4))
def test_config2_small_batch_full_size(name, b):
    # configs[2]: M in {2,4,8,16}, 1 % of the channels scaled by 20, 3 and 4 bits
    n, k = LLAMA8B[name]
    lay = G.Layer(n, k, b, 128, seed=100 + b)
    for m in (2, 4, 8, 16):
        assert _lib.describe_plan(b, 128, n, k, m, True) == SMALL_BATCH_PLANS[name][m].format(b=b, r=4 if b <= 3 else 2)
        x = o.make_activations(m, k, seed=m, outlier_frac=0.01, outlier_gain=20.0)
        y = lay.run(x)
        G.assert_close_to_oracle(y, x, lay.w, f"{name} b={b} M={m}")
        G.assert_regression_bound(y, x, lay.w, f"{name} b={b} M={m}")


@pytest.mark.parametrize("name,plan", [("gate_up", "prefill b4 g128 zp1 cfg0"), ("down", "prefill b4 g128 zp1 cfg0")])
def test_config4_prefill_full_size(name, plan):
    # configs[4]: the two largest Llama-3-70B layers at M = 2048 (gate_up: seven rounds of 512
    # workgroups and 235 MB of output; down: 224 K tiles, the longest walk of the ring)
    n, k = LLAMA70B[name]
    m = 2048
    assert _lib.describe_plan(4, 128, n, k, m, True) == plan
    q, s, z = o.make_layer(n, k, 128, seed=7)
    x = o.make_activations(m, k, seed=11)
    packed = G.pack_device(q, 4, True)
    sc, zr = G.reorder_device(s, n, k, 128), G.reorder_device(z, n, k, 128)
    y = G.gemm(4, 128, n, k, G.to_dev(x), packed, sc, zr)
    torch.cuda.synchronize()
    # two batch rows of every 128-row activation tile, at varying positions inside the tile
    rows = np.array([t * 128 + (37 * t + 5) % 128 for t in range(16)] + [t * 128 + (91 * t + 64) % 128 for t in range(16)])
    yr = y[torch.from_numpy(rows).to(G.DEV)].cpu().numpy()
    assert bool(torch.isfinite(y.float()).all())
    ref, bound = G.oracle_product_in_chunks(q, s, z, 4, 128, x[rows])
    G.assert_close_to_reference(yr, ref, bound, f"70B {name} prefill")


@pytest.mark.parametrize("name,m,plan", [("o", 512, "prefill b4 g128 zp1 cfg10"), ("o", 1024, "prefill b4 g128 zp1 cfg11"),
                                         ("down", 500, "prefill b4 g128 zp1 cfg10"), ("down", 1000, "prefill b4 g128 zp1 cfg11"),
                                         ("qkv", 512, "prefill b4 g128 zp1 cfg13"), ("qkv", 1000, "prefill b4 g128 zp1 cfg14"),
                                         ("gate_up", 512, "prefill b4 g128 zp1 cfg15"),
                                         ("o", 250, "prefill b4 g128 zp1 cfg16"), ("down", 250, "prefill b4 g128 zp1 cfg16")])
def test_medium_batch_split_tiles_full_size(name, m, plan):
    # batches of a few hundred rows on the Llama-3-70B layers: the ring tiles with K split inside a
    # workgroup of eight waves (128 x 128, 128 x 256, and 128 x 192 on qkv; down: 112 K tiles per group of
    # waves; ragged M), both tile widths in one launch (qkv at about a thousand rows), the wide tile
    # with a last round of 128 x 192 tiles (gate_up), and 64 x 128 tiles with K split (250 rows)
    n, k = LLAMA70B[name]
    assert _lib.describe_plan(4, 128, n, k, m, True) == plan
    q, s, z = o.make_layer(n, k, 128, seed=17)
    x = o.make_activations(m, k, seed=m)
    packed = G.pack_device(q, 4, True)
    sc, zr = G.reorder_device(s, n, k, 128), G.reorder_device(z, n, k, 128)
    y = G.gemm(4, 128, n, k, G.to_dev(x), packed, sc, zr)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(y.float()).all())
    tiles = (m + 63) // 64  # a row of every 64: one or two per activation tile
    rows = np.array(sorted({min(t * 64 + (37 * t + 5) % 64, m - 1) for t in range(tiles)} | {0, m - 1}))
    yr = y[torch.from_numpy(rows).to(G.DEV)].cpu().numpy()
    ref, bound = G.oracle_product_in_chunks(q, s, z, 4, 128, x[rows])
    G.assert_close_to_reference(yr, ref, bound, f"70B {name} M={m}")


@pytest.mark.parametrize("name,m,plan", [("gate_up", 512, "prefill b4 g128 zp1 cfg17"), ("gate_up", 760, "prefill b4 g128 zp1 cfg15"),
                                         ("o", 500, "prefill b4 g128 zp1 cfg16"), ("down", 512, "prefill b4 g128 zp1 cfg16")])
def test_medium_batch_llama3_8b_full_size(name, m, plan):
    # batches of a few hundred rows on the Llama-3-8B layers: 128 x 256 and 128 x 192 tiles in one round
    # (gate_up at 512 rows), the wide tile with 216 tiles of 192 rows behind its one round (760 rows), and
    # 64 x 128 tiles with K split in the workgroup (o; down: 56 K tiles per group of waves)
    n, k = LLAMA8B[name]
    assert _lib.describe_plan(4, 128, n, k, m, True) == plan
    q, s, z = o.make_layer(n, k, 128, seed=19)
    x = o.make_activations(m, k, seed=m)
    packed = G.pack_device(q, 4, True)
    sc, zr = G.reorder_device(s, n, k, 128), G.reorder_device(z, n, k, 128)
    y = G.gemm(4, 128, n, k, G.to_dev(x), packed, sc, zr)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(y.float()).all())
    tiles = (m + 63) // 64
    rows = np.array(sorted({min(t * 64 + (37 * t + 5) % 64, m - 1) for t in range(tiles)} | {0, m - 1}))
    yr = y[torch.from_numpy(rows).to(G.DEV)].cpu().numpy()
    ref, bound = G.oracle_product_in_chunks(q, s, z, 4, 128, x[rows])
    G.assert_close_to_reference(yr, ref, bound, f"8B {name} M={m}")


@pytest.mark.parametrize("m", (1, 2, 4))
def test_llama3_70b_down_decode_full_size(m):
    # 224 K tiles per row block: sixteen waves walk three and a half rounds
    n, k = LLAMA70B["down"]
    q, s, z = o.make_layer(n, k, 128, seed=3)
    x = o.make_activations(m, k, seed=m)
    packed = G.pack_device(q, 4, True)
    sc, zr = G.reorder_device(s, n, k, 128), G.reorder_device(z, n, k, 128)
    assert _lib.describe_plan(4, 128, n, k, m, True) == f"gemv b4 g128 zp1 T4 R{1 if m <= 2 else 2} W16 pad0"
    y = G.gemm(4, 128, n, k, G.to_dev(x), packed, sc, zr).cpu().numpy()
    ref, bound = G.oracle_product_in_chunks(q, s, z, 4, 128, x)
    G.assert_close_to_reference(y, ref, bound, f"70B down M={m}")
    # the decode kernel on the same layer stages the activations in chunks with a ragged last one
    # (224 tiles in chunks of 120 and 104)
    flags = 1 | (1 << 16)
    assert _lib.describe_plan(4, 128, n, k, m, True, flags).startswith("decode-chunked")
    y = G.gemm(4, 128, n, k, G.to_dev(x), packed, sc, zr, flags=flags).cpu().numpy()
    G.assert_close_to_reference(y, ref, bound, f"70B down M={m}, decode kernel")


@pytest.mark.parametrize("k_tiles,m", [(100, 16), (37, 16), (113, 9)])
def test_chunked_staging_with_a_ragged_last_chunk(k_tiles, m):
    # chunk length kc does not divide the K tiles, nor does the number of waves
    n, k = 64, 128 * k_tiles
    flags = 1 | (1 << 8)
    lay = G.Layer(n, k, 4, 128, seed=k_tiles)
    x = o.make_activations(m, k, seed=m)
    plan = _lib.describe_plan(4, 128, n, k, m, True, flags)
    if k_tiles > 60:
        assert plan.startswith("decode-chunked"), plan
    y = lay.run(x, flags=flags)
    G.assert_close_to_oracle(y, x, lay.w, plan)
    G.assert_regression_bound(y, x, lay.w, plan)


def test_config3_llama3_8b_block_through_the_plugin():
    # configs[3] at its stated layer shape: one Llama-3-8B-shaped block (hidden 4096, ffn 14336,
    # 32 heads, 8 KV heads), every linear at its own bitwidth, built by the vLLM quantisation
    # method, against the same block with dense oracle weights
    from matgptq_amd import decoder as D

    cfg = D.DecoderConfig(hidden=4096, ffn=14336, layers=1, heads=32, kv_heads=8, vocab=4096)
    dec, bits, masters = D.random_mixnmatch_decoder(cfg, 96, (2, 3, 4, 6, 8), seed=6, keep_master=True, via_plugin=True)
    assert len(set(bits.values())) >= 3

    class Dense(torch.nn.Module):
        def __init__(self, w):
            super().__init__()
            self.w = torch.from_numpy(w).cuda()  # fp16 oracle weight

        def forward(self, x):
            return (x.float() @ self.w.float().T).to(x.dtype)

    lin = {}
    for name in cfg.linear_shapes():
        codes, scale, zero = masters[f"blocks.0.{name}"]
        lin[name] = Dense(o.dequantize(codes.cpu().numpy(), scale.cpu().numpy(), zero.cpu().numpy(),
                                       bits[f"blocks.0.{name}"], cfg.group_size))
    ref = D.Decoder(cfg, [D.Block(cfg, lin, torch.float16, "cuda")], dec.embed.data, dec.head.data, dec.max_context)
    prompt = torch.randint(0, cfg.vocab, (40,), device="cuda", generator=torch.Generator(device="cuda").manual_seed(1))
    pos = torch.arange(40, device="cuda")
    a = dec(prompt, pos, dec.new_cache())
    b = ref(prompt, pos, ref.new_cache())
    assert float((a - b).abs().max()) <= 1e-2 * float(b.abs().max())
    # decode (M = 1, the gemv kernel at each layer's bitwidth) continues the prefill (M = 39)
    s = D.DecodeSession(dec)
    s.prefill(prompt[:39])
    s.token.copy_(prompt[39:40])
    s.step()
    assert float((s.logits - b).abs().max()) <= 1e-2 * float(b.abs().max())
    # every linear of the block on its own, at batch 1, against the oracle
    blk = dec.blocks[0]
    for name, (n, k) in cfg.linear_shapes().items():
        codes, scale, zero = masters[f"blocks.0.{name}"]
        w = o.dequantize(codes.cpu().numpy(), scale.cpu().numpy(), zero.cpu().numpy(), bits[f"blocks.0.{name}"], 128)
        x = o.make_activations(1, k, seed=k % 97)
        y = getattr(blk, name)(torch.from_numpy(x).cuda()).cpu().numpy()
        G.assert_close_to_oracle(y, x, w, f"block linear {name} b={bits[f'blocks.0.{name}']}")


def test_config3_full_size_decoder_graph_replays_and_every_distinct_linear():
    # configs[3] as stated: 32 blocks of Llama-3-8B's shape, vocabulary 128256, context 512, batch 1,
    # every linear at a seeded bitwidth from {2,3,4,6,8}, built through the vLLM quantisation method.
    # (i) eight decode steps replayed from the HIP graph equal the same steps run eagerly, logits and
    # tokens bit for bit; (ii) one linear of every distinct (shape, bitwidth) pair against the oracle
    # at batch 1.
    from matgptq_amd import decoder as D

    cfg = D.DecoderConfig()
    assert (cfg.hidden, cfg.ffn, cfg.layers, cfg.heads, cfg.kv_heads, cfg.vocab) == (4096, 14336, 32, 32, 8, 128256)
    context = 512
    dec, bits, masters = D.random_mixnmatch_decoder(cfg, context + 24, (2, 3, 4, 6, 8), seed=0, keep_master=True,
                                                    via_plugin=True)
    assert len(bits) == 128 and set(bits.values()) == {2, 3, 4, 6, 8}
    prompt = torch.randint(0, cfg.vocab, (context,), device="cuda", generator=torch.Generator(device="cuda").manual_seed(0))
    eager = D.DecodeSession(dec)
    eager.prefill(prompt)
    graphed = D.DecodeSession(dec)
    graphed.prefill(prompt)
    assert torch.isfinite(eager.logits).all()
    assert torch.equal(eager.logits, graphed.logits)
    graphed.capture()
    for i in range(8):
        eager.step()
        graphed.replay()
        torch.cuda.synchronize()
        assert torch.equal(eager.logits, graphed.logits), f"replay {i}"
        assert torch.equal(eager.token, graphed.token), f"replay {i}"
        assert int(graphed.pos.item()) == context + 1 + i
    del eager, graphed
    seen = set()
    for full, b in bits.items():
        _, blk, name = full.split(".")
        if (name, b) in seen:
            continue
        seen.add((name, b))
        codes, scale, zero = masters[full]
        n, k = codes.shape
        x = o.make_activations(1, k, seed=b + n % 89)
        y = getattr(dec.blocks[int(blk)], name)(torch.from_numpy(x).cuda()).cpu().numpy()
        ref, bound = G.oracle_product_in_chunks(codes.cpu().numpy(), scale.cpu().numpy(), zero.cpu().numpy(), b,
                                                cfg.group_size, x)
        G.assert_close_to_reference(y, ref, bound, f"configs[3] {full} b={b}")
    assert len(seen) >= 16  # 4 shapes x 5 bitwidths, nearly all of them drawn among 128 linears


def test_prefill_zero_point_form_deviation_per_weight():
    # The prefill kernels' zero-point form computes fma(c - 2^(b-1), scale 2^(8-b), -fp16(scale (zero - 128)))
    # while dequantize() rounds scale * fp16((c << (8-b)) - zero) once.  Bound of the difference per
    # weight: one fp16 rounding of a term no larger than 128 scale plus one of the weight itself.
    # Extract the kernel's effective weights with unit activations (X = identity block).
    n, k, b = 64, 256, 4
    lay = G.Layer(n, k, b, 128, seed=21)
    x = np.zeros((k, k), dtype=np.float16)
    x[np.arange(k), np.arange(k)] = 1.0
    y = lay.run(x)  # M = 256 rows: prefill kernel; y[j, i] = effective w[i, j]
    assert _lib.describe_plan(b, 128, n, k, k, True).split()[0] in ("prefill", "midbatch")
    w_eff = y.T.astype(np.float64)
    w = lay.w.astype(np.float64)
    s = np.repeat(lay.s.astype(np.float64), 128, axis=1)
    ulp_w = np.maximum(np.abs(w), 2.0 ** -14) * 2.0 ** -10
    ulp_term = 128.0 * s * 2.0 ** -11
    assert np.all(np.abs(w_eff - w) <= ulp_w + ulp_term + 1e-12)


@pytest.mark.parametrize("b,g,plan", [(4, 32, "prefill b4 g32 zp1 cfg3"), (8, 32, "prefill b8 g32 zp1 cfg3"),
                                      (4, -1, "prefill b4 g-1 zp1 cfg0")])
def test_prefill_other_group_sizes_full_size(b, g, plan):
    # the Llama-3-70B o layer at M = 2048 with a scale and a zero per 32 columns (kept off the tile
    # whose registers they do not fit) and per row
    n, k = LLAMA70B["o"]
    m = 2048
    assert _lib.describe_plan(b, g, n, k, m, True) == plan
    q, s, z = o.make_layer(n, k, g, seed=17)
    x = o.make_activations(m, k, seed=12)
    packed = G.pack_device(q, b, True)
    sc, zr = G.reorder_device(s, n, k, g), G.reorder_device(z, n, k, g)
    y = G.gemm(b, g, n, k, G.to_dev(x), packed, sc, zr)
    torch.cuda.synchronize()
    rows = np.array([t * 128 + (37 * t + 5) % 128 for t in range(16)])
    yr = y[torch.from_numpy(rows).to(G.DEV)].cpu().numpy()
    assert bool(torch.isfinite(y.float()).all())
    ref, bound = G.oracle_product_in_chunks(q, s, z, b, g, x[rows])
    G.assert_close_to_reference(yr, ref, bound, f"70B o prefill b={b} g={g}")
