"""The fused decode-time operators between the linears (include/matgptq_glue.h) against the torch
operators they replace, and the decoder step built from them against the step built from torch
operators.  Floating point: each operator rounds once where the torch sequence rounds two or
three times, so results agree within a few fp16 steps; the tolerances are written at each test."""
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _gen(seed):
    return torch.Generator(device=DEV).manual_seed(seed)


@pytest.mark.parametrize("with_delta", (False, True))
@pytest.mark.parametrize("m,hidden", [(1, 4096), (5, 256), (16, 8192), (3, 1000)])
def test_add_rmsnorm(m, hidden, with_delta):
    from matgptq_amd import _glue

    g = _gen(hidden + m)
    h = torch.randn(m, hidden, device=DEV, generator=g).half()
    delta = torch.randn(m, hidden, device=DEV, generator=g).half() if with_delta else None
    w = (torch.rand(hidden, device=DEV, generator=g) + 0.5).half()
    h_ref = h + delta if with_delta else h.clone()
    ref = torch.nn.functional.rms_norm(h_ref.float(), (hidden,), w.float(), 1e-5)
    x = torch.empty_like(h)
    _glue.add_rmsnorm(h, delta, w, x, 1e-5)
    assert torch.equal(h, h_ref)  # the residual sum is the same single fp16 rounding
    assert float((x.float() - ref).abs().max()) <= 2e-3 * float(ref.abs().max())  # one fp16 rounding of the result


def _rotate_ref(t, cos, sin):
    half = t.shape[-1] // 2
    rot = torch.cat((-t[..., half:], t[..., :half]), dim=-1)
    return t * cos[:, None, :] + rot * sin[:, None, :]


@pytest.mark.parametrize("m,heads,kv,d", [(1, 32, 8, 128), (4, 4, 2, 128), (2, 6, 6, 64)])
def test_rope_cache(m, heads, kv, d):
    from matgptq_amd import _glue

    g = _gen(m * heads)
    ctx = 40
    qkv = torch.randn(m, (heads + 2 * kv) * d, device=DEV, generator=g).half()
    ang = torch.rand(ctx, d, device=DEV, generator=g) * 6.28
    cos, sin = ang.cos().half(), ang.sin().half()
    pos = torch.tensor([7, 0, 39, 12][:m], device=DEV)
    k_cache = torch.randn(kv, ctx, d, device=DEV, generator=g).half()
    v_cache = torch.randn(kv, ctx, d, device=DEV, generator=g).half()
    k_ref, v_ref = k_cache.clone(), v_cache.clone()
    t = qkv.view(m, heads + 2 * kv, d).float()
    rot = _rotate_ref(t[:, :heads + kv], cos[pos].float(), sin[pos].float())
    k_ref[:, pos] = rot[:, heads:].transpose(0, 1).half()
    v_ref[:, pos] = t[:, heads + kv:].transpose(0, 1).half()
    _glue.rope_cache(qkv, cos, sin, pos, k_cache, v_cache, heads, kv)
    out = qkv.view(m, heads + 2 * kv, d)
    assert torch.equal(out[:, heads:], t[:, heads:].half())  # keys and values in qkv are left alone
    assert torch.equal(v_cache, v_ref)
    # fp32 arithmetic, one rounding: equal to the rounded fp32 reference up to one fp16 step
    assert float((out[:, :heads].float() - rot[:, :heads]).abs().max()) <= 4e-3
    assert float((k_cache.float() - k_ref.float()).abs().max()) <= 4e-3
    untouched = torch.ones(ctx, dtype=torch.bool, device=DEV)
    untouched[pos] = False
    assert torch.equal(k_cache[:, untouched], k_ref[:, untouched])


@pytest.mark.parametrize("m,heads,kv,ctx,positions", [(1, 32, 8, 600, [511]), (3, 4, 2, 64, [0, 17, 63]),
                                                      (2, 8, 8, 8192, [8191, 300]), (16, 4, 1, 100, list(range(16)))])
def test_attention(m, heads, kv, ctx, positions):
    from matgptq_amd import _glue

    d = 128
    g = _gen(ctx + m)
    qkv = torch.randn(m, (heads + 2 * kv) * d, device=DEV, generator=g).half()
    k_cache = torch.randn(kv, ctx, d, device=DEV, generator=g).half()
    v_cache = torch.randn(kv, ctx, d, device=DEV, generator=g).half()
    pos = torch.tensor(positions, device=DEV)
    out = torch.full((m, heads * d), float("nan"), device=DEV, dtype=torch.float16)
    # rows no query may see hold NaN for the kernel (it reads some of them, and must not use them)
    k_dirty, v_dirty = k_cache.clone(), v_cache.clone()
    k_dirty[:, max(positions) + 1:] = float("nan")
    v_dirty[:, max(positions) + 1:] = float("nan")
    _glue.attention(qkv, k_dirty, v_dirty, pos, out, heads, kv)
    q = qkv.view(m, heads + 2 * kv, d)[:, :heads].float()
    rep = heads // kv
    k = k_cache.float().repeat_interleave(rep, dim=0)  # [heads, ctx, d]
    v = v_cache.float().repeat_interleave(rep, dim=0)
    scores = torch.einsum("mhd,htd->mht", q, k) * d ** -0.5
    mask = torch.arange(ctx, device=DEV)[None, None, :] > pos[:, None, None]
    ref = torch.einsum("mht,htd->mhd", torch.softmax(scores.masked_fill(mask, float("-inf")), dim=-1), v)
    err = float((out.view(m, heads, d).float() - ref).abs().max())
    assert err <= 2e-3 * max(1.0, float(ref.abs().max()))  # fp32 throughout, one fp16 rounding of the result


@pytest.mark.parametrize("heads,kv,ctx,position", [(32, 8, 600, 511), (4, 2, 64, 0), (8, 8, 1000, 999), (4, 1, 300, 64)])
def test_rope_attention_equals_the_two_launches(heads, kv, ctx, position):
    from matgptq_amd import _glue

    d = 128
    g = _gen(ctx + heads)
    qkv = torch.randn(1, (heads + 2 * kv) * d, device=DEV, generator=g).half()
    ang = torch.rand(ctx, d, device=DEV, generator=g) * 6.28
    cos, sin = ang.cos().half(), ang.sin().half()
    pos = torch.tensor([position], device=DEV)
    k_cache = torch.randn(kv, ctx, d, device=DEV, generator=g).half()
    v_cache = torch.randn(kv, ctx, d, device=DEV, generator=g).half()
    k_cache[:, position + 1:] = float("nan")
    v_cache[:, position + 1:] = float("nan")
    qkv_two, k_two, v_two = qkv.clone(), k_cache.clone(), v_cache.clone()
    out_two = torch.empty(1, heads * d, device=DEV, dtype=torch.float16)
    _glue.rope_cache(qkv_two, cos, sin, pos, k_two, v_two, heads, kv)
    _glue.attention(qkv_two, k_two, v_two, pos, out_two, heads, kv)
    qkv_one, k_one, v_one = qkv.clone(), k_cache.clone(), v_cache.clone()
    out_one = torch.full((1, heads * d), float("nan"), device=DEV, dtype=torch.float16)
    _glue.rope_attention(qkv_one, cos, sin, pos, k_one, v_one, out_one, heads, kv)
    # same arithmetic in the same order: the same bits
    assert torch.equal(out_one, out_two)
    assert torch.equal(k_one[:, :position + 1], k_two[:, :position + 1])
    assert torch.equal(v_one[:, :position + 1], v_two[:, :position + 1])
    assert torch.equal(qkv_one, qkv)  # read only
    assert torch.isnan(k_one[:, position + 1:]).all() and torch.isnan(v_one[:, position + 1:]).all()


@pytest.mark.parametrize("m,heads,kv,ctx,positions", [(1, 32, 8, 600, [511]), (3, 4, 2, 64, [0, 17, 63]),
                                                      (2, 8, 8, 8192, [8191, 300]), (16, 8, 1, 100, list(range(16))),
                                                      (1, 4, 2, 65, [64]), (2, 2, 1, 130, [5, 129])])
def test_attention_split_agrees_with_the_unsplit_kernel(m, heads, kv, ctx, positions):
    from matgptq_amd import _glue

    d = 128
    g = _gen(ctx + m + heads)
    qkv = torch.randn(m, (heads + 2 * kv) * d, device=DEV, generator=g).half()
    k_cache = torch.randn(kv, ctx, d, device=DEV, generator=g).half()
    v_cache = torch.randn(kv, ctx, d, device=DEV, generator=g).half()
    k_cache[:, max(positions) + 1:] = float("nan")
    v_cache[:, max(positions) + 1:] = float("nan")
    pos = torch.tensor(positions, device=DEV)
    ref = torch.empty(m, heads * d, device=DEV, dtype=torch.float16)
    _glue.attention(qkv, k_cache, v_cache, pos, ref, heads, kv)
    ws = _glue.attention_workspace(m, heads, ctx, DEV)
    for _ in range(2):
        ws.fill_(float("nan"))  # nothing may be read from the workspace that this call did not write
        out = torch.full((m, heads * d), float("nan"), device=DEV, dtype=torch.float16)
        _glue.attention_split(qkv, None, None, pos, k_cache, v_cache, out, ws, heads, kv, fuse_rotary=False)
        # fp32 sums in another order, one fp16 rounding of the result
        assert float((out.float() - ref.float()).abs().max()) <= 2e-3 * max(1.0, float(ref.float().abs().max()))


@pytest.mark.parametrize("heads,kv,ctx,position", [(32, 8, 600, 511), (4, 2, 64, 0), (8, 8, 1000, 999), (8, 1, 300, 64),
                                                   (4, 2, 200, 127), (4, 2, 200, 128)])
def test_attention_split_with_rotary_equals_the_two_launches(heads, kv, ctx, position):
    from matgptq_amd import _glue

    d = 128
    g = _gen(ctx + heads)
    qkv = torch.randn(1, (heads + 2 * kv) * d, device=DEV, generator=g).half()
    ang = torch.rand(ctx, d, device=DEV, generator=g) * 6.28
    cos, sin = ang.cos().half(), ang.sin().half()
    pos = torch.tensor([position], device=DEV)
    k_cache = torch.randn(kv, ctx, d, device=DEV, generator=g).half()
    v_cache = torch.randn(kv, ctx, d, device=DEV, generator=g).half()
    k_cache[:, position + 1:] = float("nan")
    v_cache[:, position + 1:] = float("nan")
    qkv_two, k_two, v_two = qkv.clone(), k_cache.clone(), v_cache.clone()
    out_two = torch.empty(1, heads * d, device=DEV, dtype=torch.float16)
    _glue.rope_cache(qkv_two, cos, sin, pos, k_two, v_two, heads, kv)
    _glue.attention(qkv_two, k_two, v_two, pos, out_two, heads, kv)
    qkv_one, k_one, v_one = qkv.clone(), k_cache.clone(), v_cache.clone()
    out_one = torch.full((1, heads * d), float("nan"), device=DEV, dtype=torch.float16)
    ws = _glue.attention_workspace(1, heads, ctx, DEV).fill_(float("nan"))
    _glue.attention_split(qkv_one, cos, sin, pos, k_one, v_one, out_one, ws, heads, kv, fuse_rotary=True)
    assert float((out_one.float() - out_two.float()).abs().max()) <= 2e-3 * max(1.0, float(out_two.float().abs().max()))
    # the cache rows are the same bits: one rotary expression in every kernel
    assert torch.equal(k_one[:, :position + 1], k_two[:, :position + 1])
    assert torch.equal(v_one[:, :position + 1], v_two[:, :position + 1])
    assert torch.equal(qkv_one, qkv)
    assert torch.isnan(k_one[:, position + 1:]).all() and torch.isnan(v_one[:, position + 1:]).all()


@pytest.mark.parametrize("m,f", [(1, 14336), (7, 512), (16, 1000)])
def test_silu_mul(m, f):
    from matgptq_amd import _glue

    gu = (torch.randn(m, 2 * f, device=DEV, generator=_gen(f)) * 3).half()
    out = torch.empty(m, f, device=DEV, dtype=torch.float16)
    _glue.silu_mul(gu, out)
    ref = torch.nn.functional.silu(gu[:, :f]) * gu[:, f:]
    # same two roundings as the torch sequence; the exponential may differ in the last place
    assert float((out.float() - ref.float()).abs().max()) <= 2e-3 * float(ref.float().abs().max())


@pytest.mark.parametrize("m,n", [(1, 128256), (1, 512), (3, 1001), (2, 7), (5, 4096 * 8 + 3)])
def test_argmax_equals_torch(m, n):
    # rows of odd length start off 16 bytes from the second row on: those are read element by element
    from matgptq_amd import _glue

    x = torch.randn(m, n, device=DEV, generator=_gen(n))
    out = torch.full((m,), -1, device=DEV, dtype=torch.int64)
    _glue.argmax(x, out)
    assert torch.equal(out, x.argmax(dim=-1))


def test_argmax_takes_the_first_of_equal_values_and_a_nan_before_any_number():
    from matgptq_amd import _glue

    n = 128256
    x = torch.zeros(3, n, device=DEV)
    x[0, 70000] = x[0, 5] = x[0, 128255] = 4.0        # ties: the first index
    x[1, 99999] = float("nan")                        # a NaN wins over +inf
    x[1, 7] = float("inf")
    x[2] = -float("inf")                              # nothing larger than the start value: index 0
    out = torch.empty(3, device=DEV, dtype=torch.int64)
    _glue.argmax(x, out)
    assert out.tolist() == [5, 99999, 0]
    assert torch.equal(out, x.argmax(dim=-1))


def test_wrong_tensors_are_refused():
    from matgptq_amd import _glue

    h = torch.zeros(1, 256, device=DEV, dtype=torch.float16)
    with pytest.raises(_glue.GlueError):
        _glue.add_rmsnorm(h.float(), None, h[0], h, 1e-5)
    with pytest.raises(_glue.GlueError):
        _glue.add_rmsnorm(h, None, h[0, :128], h, 1e-5)
    with pytest.raises(_glue.GlueError):
        _glue.silu_mul(h, torch.zeros(1, 100, device=DEV, dtype=torch.float16))
    with pytest.raises(_glue.GlueError):
        _glue.argmax(h, torch.zeros(1, device=DEV, dtype=torch.int64))          # fp16 logits
    with pytest.raises(_glue.GlueError):
        _glue.argmax(h.float(), torch.zeros(2, device=DEV, dtype=torch.int64))  # one index per row


def _decoder(context=80, seed=5):
    from matgptq_amd import decoder as D

    cfg = D.DecoderConfig(hidden=512, ffn=1024, layers=2, heads=4, kv_heads=2, vocab=512)  # head dimension 128
    dec, _, _ = D.random_mixnmatch_decoder(cfg, context, (2, 3, 4, 6, 8), seed=seed)
    return D, cfg, dec


@pytest.mark.parametrize("context", (80, 1100))  # short cache: one attention launch; long: split over workgroups
@pytest.mark.parametrize("rows", (1, 3))
def test_fused_step_matches_step_of_torch_operators(rows, context):
    D, cfg, dec = _decoder(context)
    assert dec.fused_applies(rows) and not dec.fused_applies(17)
    assert dec.split_attention == (context > 768)
    prompt = torch.randint(0, cfg.vocab, (30,), device=DEV, generator=_gen(1))
    cache = dec.new_cache()
    dec(prompt, torch.arange(30, device=DEV), cache)  # 30 rows: torch operators
    tokens = torch.randint(0, cfg.vocab, (rows,), device=DEV, generator=_gen(2))
    pos = torch.arange(30, 30 + rows, device=DEV)
    cache_a, cache_b = cache.clone(), cache.clone()
    a = dec(tokens, pos, cache_a)
    dec.fused = False
    b = dec(tokens, pos, cache_b)
    dec.fused = True
    # two fp16 pipelines over two blocks
    assert float((a - b).abs().max()) <= 2e-2 * float(b.abs().max())
    assert float((cache_a.float() - cache_b.float()).abs().max()) <= 2e-2 * float(cache_b.float().abs().max())
    assert torch.equal(cache_a[:, :, :, 30 + rows:], cache[:, :, :, 30 + rows:])  # later rows untouched


def test_graph_replays_equal_eager_fused_steps():
    D, cfg, dec = _decoder()
    prompt = torch.randint(0, cfg.vocab, (24,), device=DEV, generator=_gen(3))
    eager = D.DecodeSession(dec).generate(prompt, 12, use_graph=False)
    s = D.DecodeSession(dec)
    graph = s.generate(prompt, 12, use_graph=True)
    assert torch.equal(eager, graph)
    again = s.generate(prompt, 12, use_graph=True)  # the captured step starts over from a new prompt
    assert torch.equal(eager, again)
