"""HIP path against the oracle, through the C ABI, on a real MI355X.

Integer results (slice, pack, unpack) and the dense dequantised weight must be
bit-exact; GEMM outputs must be within the tolerance stated in tests/_gpu_util.py.
"""
import numpy as np
import pytest
import torch

from matgptq_amd import _lib
from oracle import matgptq_oracle as o
from tests import _gpu_util as G

pytestmark = pytest.mark.gpu
BITS = (2, 3, 4, 6, 8)
GROUPS = (128, 32, -1)
DECODE_KERNEL = 1 | (1 << 8)  # flags: asynchronous, decode kernel forced (one row block per wave, eight K slices)


@pytest.mark.parametrize("b", BITS)
def test_slice_pack_unpack_bit_exact(b):
    L = G.lib()
    rng = np.random.default_rng(b)
    n, k = 80, 640
    q = rng.integers(0, 256, (n, k), dtype=np.uint8)
    q[0, :256] = np.arange(256, dtype=np.uint8)  # every master code appears
    ref = o.slice_codes(q, b)
    qd = G.to_dev(q)
    sl = torch.empty_like(qd)
    _lib.check(L.matgptq_slice_device(qd.data_ptr(), q.size, b, sl.data_ptr(), G.stream()))
    assert np.array_equal(sl.cpu().numpy(), ref)
    # device pack (slicing in registers) == host pack, word for word
    host = np.zeros(L.matgptq_packed_words(b, n, k), dtype=np.uint32)
    _lib.check(L.matgptq_pack_host(q.ctypes.data, n, k, b, 1, host.ctypes.data))
    dev = G.pack_device(q, b, from_master=True)
    assert np.array_equal(dev.cpu().numpy().view(np.uint32), host)
    assert np.array_equal(G.pack_device(ref, b, from_master=False).cpu().numpy().view(np.uint32), host)
    # the codes the GEMM kernels see (device unpack uses their unpack sequence)
    back = torch.full((n, k), 255, dtype=torch.uint8, device=G.DEV)
    _lib.check(L.matgptq_unpack_device(dev.data_ptr(), n, k, b, back.data_ptr(), G.stream()))
    assert np.array_equal(back.cpu().numpy(), ref)


def test_slice_device_odd_length():
    L = G.lib()
    q = np.arange(1003, dtype=np.int64).astype(np.uint8)
    qd = G.to_dev(q)
    out = torch.zeros_like(qd)
    _lib.check(L.matgptq_slice_device(qd.data_ptr(), q.size, 3, out.data_ptr(), G.stream()))
    assert np.array_equal(out.cpu().numpy(), o.slice_codes(q, 3))
    _lib.check(L.matgptq_slice_device(None, 0, 3, None, G.stream()))  # empty input is a no-op


@pytest.mark.parametrize("g", GROUPS)
@pytest.mark.parametrize("b", BITS)
def test_dequantize_bit_exact(b, g, golden):
    L = G.lib()
    lay = G.Layer(48, 512, b, g, seed=10 + b)
    w = torch.full((48, 512), float("nan"), dtype=torch.float16, device=G.DEV)
    _lib.check(L.matgptq_dequantize_device(b, g, 48, 512, lay.packed.data_ptr(), lay.scales.data_ptr(),
                                           lay.zeros.data_ptr(), w.data_ptr(), G.stream()))
    assert np.array_equal(w.cpu().numpy().view(np.uint16), lay.w.view(np.uint16))
    if g == 128:  # and against the vectors the reference's own dequantize produced
        n, k = golden["q"].shape
        pk = G.pack_device(golden["q"], b, True)
        sd, zd = G.reorder_device(golden["scale"], n, k, g), G.reorder_device(golden["zero"], n, k, g)
        w = torch.full((n, k), float("nan"), dtype=torch.float16, device=G.DEV)
        _lib.check(L.matgptq_dequantize_device(b, g, n, k, pk.data_ptr(), sd.data_ptr(), zd.data_ptr(),
                                               w.data_ptr(), G.stream()))
        assert np.array_equal(w.cpu().numpy().view(np.uint16), golden[f"w_b{b}"].view(np.uint16))


@pytest.mark.parametrize("b", BITS)
def test_forward_against_reference_vectors(b, golden):
    # FakeMatryoshkaLinear.forward of the reference on its own small layer (M = 3 -> decode path)
    n, k = golden["q"].shape
    pk = G.pack_device(golden["q"], b, True)
    sd, zd = G.reorder_device(golden["scale"], n, k, 128), G.reorder_device(golden["zero"], n, k, 128)
    y = G.gemm(b, 128, n, k, G.to_dev(golden["x"]), pk, sd, zd).cpu().numpy()
    ref = golden[f"y_b{b}"].astype(np.float64)
    assert np.max(np.abs(y - ref)) <= G.REL_TOL * np.max(np.abs(ref))
    G.assert_close_to_oracle(y, golden["x"], golden[f"w_b{b}"], f"golden b={b}")


@pytest.mark.parametrize("zp", (False, True))
@pytest.mark.parametrize("g", GROUPS)
@pytest.mark.parametrize("b", BITS)
def test_decode_parity(b, g, zp):
    # the default choice (from some batch size on the mid-batch kernel) and the decode kernel forced
    lay = G.Layer(64, 1024, b, g, seed=b, zero_points=zp)
    for m in (1, 2, 3, 5, 8, 16):
        x = o.make_activations(m, 1024, seed=m)
        G.assert_close_to_oracle(lay.run(x), x, lay.w, f"small batch b={b} g={g} zp={zp} M={m}")
        G.assert_close_to_oracle(lay.run(x, flags=DECODE_KERNEL), x, lay.w, f"decode b={b} g={g} zp={zp} M={m}")
    assert _lib.describe_plan(b, g, 64, 1024, 16, zp, DECODE_KERNEL).startswith("decode")


@pytest.mark.parametrize("zp", (False, True))
@pytest.mark.parametrize("g", GROUPS)
@pytest.mark.parametrize("b", BITS)
def test_prefill_parity(b, g, zp):
    lay = G.Layer(336, 512, b, g, seed=20 + b, zero_points=zp)  # 21 row blocks: ragged workgroups
    for m in (17, 64, 100, 257):
        x = o.make_activations(m, 512, seed=m)
        G.assert_close_to_oracle(lay.run(x), x, lay.w, f"prefill b={b} g={g} zp={zp} M={m}")


def _tile(cfg):
    # flags that force prefill tile configuration `cfg`: 64 + cfg up to 15, 89 for configuration 16
    return 1 | ((64 + cfg if cfg < 16 else 89 + cfg - 16) << 8)


@pytest.mark.parametrize("cfg", range(18))
def test_prefill_every_tile_configuration(cfg):
    lay = G.Layer(1040, 1024, 4, 128, seed=3)
    x = o.make_activations(300, 1024, seed=1)
    G.assert_close_to_oracle(lay.run(x, flags=_tile(cfg)), x, lay.w, f"cfg {cfg}")
    assert _lib.describe_plan(4, 128, 1040, 1024, 300, True, _tile(cfg)).endswith(f"cfg{cfg}")


def _decode_variants():
    return [1 | (v << 8) | (flavour << 16) for v in range(1, 43) for flavour in (1, 2)]


@pytest.mark.parametrize("zp", (False, True))
@pytest.mark.parametrize("g", GROUPS)
@pytest.mark.parametrize("b", BITS)
def test_prefill_ring_tile_every_format(b, g, zp):
    # the 128 x 256 tile counts its loads in flight by hand, and the count depends on the
    # bitwidth (one or two code segments), the group size and the zero points; ragged M and N,
    # odd number of K tiles
    n, k, m = 304, 128 * 7, 200
    lay = G.Layer(n, k, b, g, seed=31 * b + (g & 7), zero_points=zp)
    x = o.make_activations(m, k, seed=b)
    for _ in range(2):
        y = lay.run(x, flags=1 | (64 << 8))
        G.assert_close_to_oracle(y, x, lay.w, f"ring tile b={b} g={g} zp={zp}")
    assert _lib.describe_plan(b, g, n, k, m, zp, 1 | (64 << 8)).endswith("cfg0")


@pytest.mark.parametrize("zp", (False, True))
@pytest.mark.parametrize("g", GROUPS)
@pytest.mark.parametrize("b", BITS)
def test_prefill_split_tiles_every_format(b, g, zp):
    # K in two halves inside a workgroup of eight waves, each group with a ring of its own and
    # the same hand-counted waits; the second group's sums cross LDS at the end.  Seven K tiles
    # (the second group walks one tile fewer), ragged M and N; every tile shape.
    n, k, m = 304, 128 * 7, 200
    lay = G.Layer(n, k, b, g, seed=29 * b + (g & 7), zero_points=zp)
    x = o.make_activations(m, k, seed=b + 2)
    for cfg in (10, 11, 13, 16):
        flags = _tile(cfg)
        for _ in range(2):
            G.assert_close_to_oracle(lay.run(x, flags=flags), x, lay.w, f"split tile cfg{cfg} b={b} g={g} zp={zp}")
        assert _lib.describe_plan(b, g, n, k, m, zp, flags).endswith(f"cfg{cfg}")


@pytest.mark.parametrize("k_tiles", (1, 2, 3, 10))
@pytest.mark.parametrize("cfg", (10, 11, 13, 16))
def test_prefill_split_tiles_short_and_even_walks(cfg, k_tiles):
    # one K tile leaves the second group with nothing but zeros; two give each group a single trip
    n, k, m = 528, 128 * k_tiles, 130
    lay = G.Layer(n, k, 4, 128, seed=k_tiles)
    x = o.make_activations(m, k, seed=cfg)
    G.assert_close_to_oracle(lay.run(x, flags=_tile(cfg)), x, lay.w, f"split cfg{cfg} {k_tiles} K tiles")


def test_prefill_split_tile_agrees_with_the_plain_tile_closely():
    # the same products in the same order within each half of K; the two halves are added in fp32
    n, k, m = 1024, 4096, 256
    lay = G.Layer(n, k, 4, 128, seed=8)
    x = o.make_activations(m, k, seed=9)
    plain = lay.run(x, flags=1 | (67 << 8)).astype(np.float64)
    for cfg in (10, 11, 13, 16):
        y = lay.run(x, flags=_tile(cfg)).astype(np.float64)
        assert np.max(np.abs(y - plain)) <= 2.0 ** -9 * np.max(np.abs(plain))
        assert np.mean(y == plain) > 0.9


def _mid_variants(b, g):
    # forced shapes of the mid-batch kernel: 80 + rsel + 3 msel (1, 2, 4 row blocks x 16, 32, 64 batch rows), and
    # 91 (eight row blocks x 32 batch rows) where the format takes it: up to 4 bits, one scale per tile or row
    return list(range(80, 89)) + ([91] if b <= 4 and g != 32 else [])


def test_midbatch_eight_row_blocks_refused_where_the_format_does_not_take_them():
    with pytest.raises(_lib.MatGPTQError):
        _lib.describe_plan(6, 128, 304, 1024, 32, True, 1 | (91 << 8))
    with pytest.raises(_lib.MatGPTQError):
        _lib.describe_plan(4, 32, 304, 1024, 32, True, 1 | (91 << 8))
    assert _lib.describe_plan(4, 128, 304, 1024, 32, True, 1 | (91 << 8)) == "midbatch b4 g128 zp1 R8 mb2"


@pytest.mark.parametrize("zp", (False, True))
@pytest.mark.parametrize("g", GROUPS)
@pytest.mark.parametrize("b", BITS)
def test_midbatch_kernel_every_format(b, g, zp):
    # K split over the eight waves of a workgroup: 13 K tiles (ragged split, odd walk), 19 row
    # blocks (ragged for 2 and 4 row blocks per workgroup), ragged batch
    n, k, m = 304, 128 * 13, 77
    lay = G.Layer(n, k, b, g, seed=17 * b + (g & 7), zero_points=zp)
    x = o.make_activations(m, k, seed=b + 1)
    for v in _mid_variants(b, g):
        flags = 1 | (v << 8)
        y = lay.run(x, flags=flags)
        G.assert_close_to_oracle(y, x, lay.w, f"mid-batch b={b} g={g} zp={zp} variant={v}")
        assert _lib.describe_plan(b, g, n, k, m, zp, flags).startswith("midbatch")


@pytest.mark.parametrize("m", (17, 32, 33, 64, 128, 250))
@pytest.mark.parametrize("n,k", [(4096, 4096), (512, 14336), (1040, 384)])
def test_midbatch_kernel_shapes(n, k, m):
    # long and short K walks (K = 384: five of the eight waves have no tile at all)
    lay = G.Layer(n, k, 4, 128, seed=n + m)
    x = o.make_activations(m, k, seed=m)
    rows = np.r_[0:min(m, 24), max(m - 24, 0):m]
    for v in _mid_variants(4, 128):
        y = lay.run(x, flags=1 | (v << 8))
        G.assert_close_to_oracle(y[rows], x[rows], lay.w, f"mid-batch {n}x{k} M={m} variant={v}")


def test_midbatch_kernel_agrees_with_prefill_tile_closely():
    # same products, different summation order (eight partial sums): outputs agree to fp32
    # rounding of the accumulation, far inside one fp16 rounding of most outputs
    n, k, m, b, g = 2048, 4096, 96, 4, 128
    lay = G.Layer(n, k, b, g, seed=5)
    x = o.make_activations(m, k, seed=6)
    a = lay.run(x, flags=1 | (81 << 8)).astype(np.float64)
    c = lay.run(x, flags=1 | (68 << 8)).astype(np.float64)
    scale = np.max(np.abs(c))
    assert np.max(np.abs(a - c)) <= 2.0 ** -9 * scale
    assert np.mean(a == c) > 0.9


def test_midbatch_kernel_outlier_channels():
    lay = G.Layer(512, 4096, 3, 128, seed=12)
    x = o.make_activations(48, 4096, seed=3, outlier_frac=0.01, outlier_gain=20.0)
    for v in _mid_variants(3, 128):
        G.assert_close_to_oracle(lay.run(x, flags=1 | (v << 8)), x, lay.w, f"outliers variant={v}")


def test_decode_every_work_split():
    # all (R, S, W) shapes in both flavours; 65 row blocks leave idle slots in the last
    # workgroup, K = 4096 gives up to 32 tiles per wave
    lay = G.Layer(1040, 4096, 4, 128, seed=4)
    x = o.make_activations(3, 4096, seed=2)
    ran = 0
    for flags in _decode_variants():
        try:
            y = lay.run(x, flags=flags)
        except _lib.MatGPTQError as e:
            assert "variant" in str(e)
            continue
        G.assert_close_to_oracle(y, x, lay.w, f"flags {flags:#x}")
        ran += 1
    assert ran >= 60


@pytest.mark.parametrize("b", (3, 4))
@pytest.mark.parametrize("m", (2, 4, 8, 16))
def test_small_batch_with_outlier_channels(b, m):
    # 1 % of the channels scaled by 20: stresses the fp32 accumulation
    lay = G.Layer(256, 4096, b, 128, seed=30 + m)
    x = o.make_activations(m, 4096, seed=m, outlier_frac=0.01, outlier_gain=20.0)
    G.assert_close_to_oracle(lay.run(x), x, lay.w, f"outliers b={b} M={m}")
    G.assert_close_to_oracle(lay.run(x, flags=DECODE_KERNEL), x, lay.w, f"outliers, decode kernel b={b} M={m}")


def test_chunked_activation_staging():
    # M = 16 with K = 14336 does not fit in LDS at once: the kernel walks K in chunks
    lay = G.Layer(64, 14336, 4, 128, seed=7)
    x = o.make_activations(16, 14336, seed=7)
    assert _lib.describe_plan(4, 128, 64, 14336, 16, True, DECODE_KERNEL).startswith("decode-chunked")
    G.assert_close_to_oracle(lay.run(x, flags=DECODE_KERNEL), x, lay.w, "chunked")
    G.assert_close_to_oracle(lay.run(x), x, lay.w, "default choice")


@pytest.mark.parametrize("gsz", (-1, 32, 128))
@pytest.mark.parametrize("m", (1, 8, 16))
@pytest.mark.parametrize("k", (1024, 4096, 8192))
@pytest.mark.parametrize("b", BITS)
def test_reference_kernel_test_grid(b, k, m, gsz):
    # the reference's own test (inference_lib/test_matgptq_matmul.py:11-49), fp16 half of
    # it: codes < 2^b, scales in {0,1}, integer activations, N = 16, symmetric form.
    # All arithmetic is exact, so the result must equal the closed form bit for bit.
    rng = np.random.default_rng(1)
    n = 16
    g = k if gsz == -1 else gsz
    codes = rng.integers(0, 1 << b, (n, k), dtype=np.uint8)
    scales = np.round(rng.random((n, k // g))).astype(np.float16)
    x = np.round(rng.standard_normal((m, k))).astype(np.float16)
    w = o.dequantize_kernel_form(codes, scales, b, gsz)
    expect = o.linear_f64(x, w).astype(np.float16)
    pk = G.pack_device(codes, b, from_master=False)
    sd = G.reorder_device(scales, n, k, gsz)
    for flags in (1, DECODE_KERNEL):
        y = G.gemm(b, gsz, n, k, G.to_dev(x), pk, sd, None, flags=flags).cpu().numpy()
        assert np.array_equal(y.view(np.uint16), expect.view(np.uint16)), flags


LLAMA8B = {"qkv": (6144, 4096), "o": (4096, 4096), "gate_up": (28672, 4096), "down": (4096, 14336)}


@pytest.mark.parametrize("name", sorted(LLAMA8B))
@pytest.mark.parametrize("b", BITS)
def test_llama3_8b_layers_decode_full_size(name, b):
    n, k = LLAMA8B[name]
    lay = G.Layer(n, k, b, 128, seed=0)
    x = o.make_activations(1, k, seed=0)
    y = lay.run(x)
    G.assert_close_to_oracle(y, x, lay.w, f"{name} b={b}")
    # linearity in x at full size: f(2x) = 2 f(x) up to the last bit of the fp16 result
    # (activations are pre-scaled by powers of two inside the kernel, so the smallest of
    # them may round differently after doubling)
    y2 = lay.run((x.astype(np.float32) * 2).astype(np.float16)).astype(np.float64)
    assert np.max(np.abs(y2 - 2.0 * y.astype(np.float64))) <= 2.0 ** -9 * np.max(np.abs(y2))


def test_llama3_70b_layer_prefill_full_size():
    n, k, m = 8192, 8192, 2048
    lay = G.Layer(n, k, 4, 128, seed=0)
    x = o.make_activations(m, k, seed=0)
    y = lay.run(x)
    rows = np.array([0, 1, 777, 2047])
    G.assert_close_to_oracle(y[rows], x[rows], lay.w, "70B o-proj prefill")
    # every row agrees with the decode kernel run on that row alone (different kernel, same answer)
    y1 = lay.run(x[5:6])
    assert np.max(np.abs(y1.astype(np.float64) - y[5:6])) <= 2e-3 * np.max(np.abs(y1.astype(np.float64)))


@pytest.mark.parametrize("zp", (True, False))
def test_prefill_paired_tiles_with_a_split_tail_odd_tile_count(zp):
    # 128 x 256 tiles two to a workgroup of eight waves, the remaining rows as 128 x 128 tiles with K
    # split inside the workgroup: 73 activation tiles x 7 whole weight tiles = 511 wide tiles (the last
    # workgroup's second tile is empty), 8 row blocks in the tail, ragged M
    n, k, m = 1920, 384, 73 * 128 - 5
    flags = 1 | ((64 + 12) << 8)
    lay = G.Layer(n, k, 4, 128, seed=12, zero_points=zp)
    x = o.make_activations(m, k, seed=12)
    y = lay.run(x, flags=flags)
    G.assert_close_to_oracle(y, x, lay.w, "paired tiles + split tail")
    G.assert_regression_bound(y, x, lay.w, "paired tiles + split tail")
    # the wide tiles run the four-wave tail kernel's arithmetic; the narrow ones add two halves of K
    y8 = lay.run(x, flags=1 | ((64 + 8) << 8))
    assert np.array_equal(y[:, :1792], y8[:, :1792])
    assert np.max(np.abs(y[:, 1792:].astype(np.float64) - y8[:, 1792:])) <= 2e-3 * np.max(np.abs(y8.astype(np.float64)))


@pytest.mark.parametrize("b,g,zp", ((4, 128, True), (4, 128, False), (2, 128, True), (3, 128, True), (8, 128, True),
                                    (6, 128, True), (4, -1, True), (4, 32, False)))
def test_prefill_two_tile_widths_in_one_launch(b, g, zp):
    # 65 row blocks, 73 activation tiles (7 slots per column): 3 tiles of 192 rows take the first 36 row
    # blocks, 4 tiles of 128 rows the other 29 (the last one ragged); ragged M.  Both parts run the
    # arithmetic of their own tile, so each equals the launch that uses that width alone.
    n, k, m = 1040, 384, 73 * 128 - 5
    lay = G.Layer(n, k, b, g, seed=14 + b, zero_points=zp)
    x = o.make_activations(m, k, seed=14)
    assert _lib.describe_plan(b, g, n, k, m, zp, 1 | ((64 + 14) << 8)).endswith("cfg14")
    y = lay.run(x, flags=1 | ((64 + 14) << 8))
    G.assert_close_to_oracle(y, x, lay.w, f"two widths b={b} g={g} zp={zp}")
    G.assert_regression_bound(y, x, lay.w, f"two widths b={b} g={g} zp={zp}")
    wide = lay.run(x, flags=1 | ((64 + 9) << 8))
    narrow = lay.run(x, flags=1 | ((64 + 3) << 8))
    assert np.array_equal(y[:, :576], wide[:, :576])
    assert np.array_equal(y[:, 576:], narrow[:, 576:])


@pytest.mark.parametrize("b,g,zp", ((4, 128, True), (4, 128, False), (2, 128, True), (8, 128, True), (6, 128, True),
                                    (4, -1, True)))
def test_prefill_wide_tiles_with_a_tail_of_192_row_tiles(b, g, zp):
    # 73 activation tiles: 7 weight tiles of 256 rows make up the whole round (511 workgroups), the other
    # 29 row blocks go to three tiles of 192 rows (the last one ragged); ragged M.  Each part equals
    # the launch that uses its width alone.
    n, k, m = 7 * 256 + 29 * 16, 384, 73 * 128 - 5
    lay = G.Layer(n, k, b, g, seed=15 + b, zero_points=zp)
    x = o.make_activations(m, k, seed=15)
    y = lay.run(x, flags=1 | ((64 + 15) << 8))
    G.assert_close_to_oracle(y, x, lay.w, f"192-row tail b={b} g={g} zp={zp}")
    G.assert_regression_bound(y, x, lay.w, f"192-row tail b={b} g={g} zp={zp}")
    wide = lay.run(x, flags=1 | ((64 + 0) << 8))
    tail = lay.run(x, flags=1 | ((64 + 9) << 8))
    assert np.array_equal(y[:, :1792], wide[:, :1792])
    assert np.array_equal(y[:, 1792:], tail[:, 1792:])


@pytest.mark.parametrize("b,g,zp", ((4, 128, True), (4, 128, False), (2, 128, True), (3, 128, True), (8, 128, True),
                                    (4, -1, True), (4, 32, False)))
def test_prefill_widest_tile_mixed_with_192_row_tiles(b, g, zp):
    # 99 row blocks, 73 activation tiles (7 slots per column): 4 tiles of 256 rows take the first 64 row
    # blocks, 3 tiles of 192 rows the other 35 (the last one ragged); ragged M.  Each part equals the
    # launch that uses its width alone.
    n, k, m = 99 * 16, 384, 73 * 128 - 5
    lay = G.Layer(n, k, b, g, seed=16 + b, zero_points=zp)
    x = o.make_activations(m, k, seed=16)
    assert _lib.describe_plan(b, g, n, k, m, zp, _tile(17)).endswith("cfg17")
    y = lay.run(x, flags=_tile(17))
    G.assert_close_to_oracle(y, x, lay.w, f"256 and 192 rows b={b} g={g} zp={zp}")
    G.assert_regression_bound(y, x, lay.w, f"256 and 192 rows b={b} g={g} zp={zp}")
    wide = lay.run(x, flags=_tile(0))
    narrow = lay.run(x, flags=_tile(9))
    assert np.array_equal(y[:, :1024], wide[:, :1024])
    assert np.array_equal(y[:, 1024:], narrow[:, 1024:])


def test_prefill_two_tile_widths_forced_where_they_do_not_apply():
    # one round of narrow tiles is enough here: the launch degenerates to those
    n, k, m = 304, 128 * 7, 200
    lay = G.Layer(n, k, 4, 128, seed=3)
    x = o.make_activations(m, k, seed=3)
    y = lay.run(x, flags=1 | ((64 + 14) << 8))
    assert np.array_equal(y, lay.run(x, flags=1 | ((64 + 3) << 8)))
    # ... and the mix of 256 and 192 rows to tiles of 192 rows
    assert np.array_equal(lay.run(x, flags=_tile(17)), lay.run(x, flags=_tile(9)))


def test_llama3_70b_qkv_at_1024_rows_takes_both_widths():
    n, k, m = 10240, 8192, 1024
    assert _lib.describe_plan(4, 128, n, k, m, True).endswith("cfg14")
    lay = G.Layer(n, k, 4, 128, seed=1)
    x = o.make_activations(m, k, seed=1)
    y = lay.run(x)
    assert np.all(np.isfinite(y))
    rows = np.array([0, 129, 1023])
    G.assert_close_to_oracle(y[rows], x[rows], lay.w, "70B qkv at M = 1024")


def test_llama3_70b_qkv_prefill_full_size_with_tail_tiles():
    # 10240 rows at M = 2048: the planner splits the launch into 128 x 256 tiles (rows below 8192, two
    # to a workgroup of eight waves) and a tail of 128 x 128 tiles with K split inside the workgroup;
    # rows of both parts against the oracle
    n, k, m = 10240, 8192, 2048
    assert _lib.describe_plan(4, 128, n, k, m, True).endswith("cfg12")
    lay = G.Layer(n, k, 4, 128, seed=0)
    x = o.make_activations(m, k, seed=0)
    y = lay.run(x)
    assert np.all(np.isfinite(y))
    rows = np.array([0, 130, 1023, 2047])
    G.assert_close_to_oracle(y[rows], x[rows], lay.w, "70B qkv prefill")
    tail = y[rows][:, 8192:].astype(np.float64)
    ref = o.linear_f64(x[rows], lay.w[8192:])
    assert np.max(np.abs(tail - ref)) <= G.REL_TOL * np.max(np.abs(ref))


def test_sync_flag_and_error_paths_on_device():
    lay = G.Layer(32, 256, 4, 128, seed=1)
    x = o.make_activations(2, 256, seed=1)
    y_async = lay.run(x, flags=1)
    y_sync = lay.run(x, flags=0)  # SYNC: the call itself waits for the kernel
    assert np.array_equal(y_async, y_sync)
    with pytest.raises(_lib.MatGPTQError, match="variant"):
        lay.run(x, flags=1 | (200 << 8))


# ---------------------------------------------------------------- bfloat16 storage (flag bit 1)

def _bf16_dev(a_f32: np.ndarray) -> torch.Tensor:
    """float32 array of bfloat16-representable values -> bfloat16 tensor on the device."""
    return torch.from_numpy(np.ascontiguousarray(a_f32, dtype=np.float32)).to(torch.bfloat16).to(G.DEV)


def _gemm_bf16(b, g, n, k, x_f32, packed, s_f32, z_f32, flags=3):
    L = G.lib()
    xd = _bf16_dev(x_f32)
    sd = _bf16_dev(s_f32)
    sr = torch.empty_like(sd)
    _lib.check(L.matgptq_reorder_scales_device(sd.data_ptr(), n, k, g, sr.data_ptr(), G.stream()))
    zr = None
    if z_f32 is not None:
        zd = _bf16_dev(z_f32)
        zr = torch.empty_like(zd)
        _lib.check(L.matgptq_reorder_scales_device(zd.data_ptr(), n, k, g, zr.data_ptr(), G.stream()))
    y = torch.full((xd.shape[0], n), float("nan"), dtype=torch.bfloat16, device=G.DEV)  # poisoned
    _lib.check(L.matgptq_gemm(b, g, n, k, xd.shape[0], packed.data_ptr(), sr.data_ptr(),
                              zr.data_ptr() if zr is not None else None, xd.data_ptr(), y.data_ptr(),
                              G.stream(), flags))
    torch.cuda.synchronize()
    return y.float().cpu().numpy()


# One bfloat16 rounding of the output is 2^-9 relative; the oracle additionally rounds every
# weight to bfloat16 (2^-9 each, independent), which the decode-regime kernels do not (they keep
# fp16 weights / exact products; the prefill kernel does round them, see the identity test below).
# Bar: max error <= 1e-2 of the largest output, as for fp16.
@pytest.mark.parametrize("b", BITS)
def test_bf16_forward_against_reference_vectors(b, golden):
    n, k = golden["q"].shape
    pk = G.pack_device(golden["q"], b, True)
    y = _gemm_bf16(b, 128, n, k, golden["x_bf16"], pk, golden["scale_bf16"], golden["zero_bf16"])
    ref = golden[f"y_bf16_b{b}"].astype(np.float64)
    assert np.all(np.isfinite(y))
    assert np.max(np.abs(y - ref)) <= G.REL_TOL * np.max(np.abs(ref))


@pytest.mark.parametrize("m", (1, 5, 16, 40, 200))
@pytest.mark.parametrize("g", GROUPS)
@pytest.mark.parametrize("b", BITS)
def test_bf16_gemm_matches_oracle(b, g, m):
    n, k = 96, 1024
    q, s16, z16 = o.make_layer(n, k, g, seed=3 * b + m)
    s = o.round_to_bf16(s16.astype(np.float32))
    z = z16.astype(np.float32)  # integers up to 255: bfloat16 values
    x = o.round_to_bf16(o.make_activations(m, k, seed=m + b, outlier_frac=0.01).astype(np.float32))
    pk = G.pack_device(q, b, True)
    for zeros in (z, None):
        zz = z if zeros is not None else np.full_like(z, 128.0)
        y = _gemm_bf16(b, g, n, k, x, pk, s, zeros)
        w = o.dequantize_bf16(q, s, zz, b, g)
        ref = o.linear_f64(x, w)
        assert np.all(np.isfinite(y))
        err = np.abs(y - ref)
        assert err.max() <= G.REL_TOL * np.max(np.abs(ref)), (b, g, m, zeros is None, err.max())
        # output values are bfloat16
        assert np.array_equal(o.round_to_bf16(y), y)


def test_bf16_small_scales_and_large_activations():
    # scales far below fp16's normal range and activations at the top of it
    n, k, b, g = 64, 512, 4, 128
    q, _, z16 = o.make_layer(n, k, g, seed=11)
    s = o.round_to_bf16(np.full((n, k // g), 3e-7, dtype=np.float32))
    z = z16.astype(np.float32)
    x = o.round_to_bf16((o.make_activations(48, k, seed=2).astype(np.float32)) * 8000.0)
    pk = G.pack_device(q, b, True)
    for rows in (slice(0, 3), slice(0, 48)):  # decode and prefill kernels
        y = _gemm_bf16(b, g, n, k, x[rows], pk, s, z)
        ref = o.linear_f64(x[rows], o.dequantize_bf16(q, s, z, b, g))
        assert np.all(np.isfinite(y))
        assert np.max(np.abs(y - ref)) <= G.REL_TOL * np.max(np.abs(ref))


@pytest.mark.parametrize("gsz", GROUPS)
@pytest.mark.parametrize("m", (1, 8, 16))
@pytest.mark.parametrize("k", (1024, 4096, 8192))
@pytest.mark.parametrize("b", BITS)
def test_reference_kernel_test_grid_bf16(b, k, m, gsz):
    # the bfloat16 half of the reference's test grid (inference_lib/test_matgptq_matmul.py:11-49):
    # every product and partial sum is an integer below 2^24, so the fp32 accumulation is exact
    # and the output must be the bfloat16 rounding of the closed form, bit for bit.
    rng = np.random.default_rng(2)
    n = 16
    g = k if gsz == -1 else gsz
    codes = rng.integers(0, 1 << b, (n, k), dtype=np.uint8)
    scales = np.round(rng.random((n, k // g))).astype(np.float32)
    x = np.round(rng.standard_normal((m, k))).astype(np.float32)
    w = (codes.astype(np.float64) - (1 << (b - 1))) * np.repeat(scales, g, axis=1) * (1 << (8 - b))
    expect = o.round_to_bf16(o.linear_f64(x, w))
    pk = G.pack_device(codes, b, from_master=False)
    for flags in (3, DECODE_KERNEL | 2):
        y = _gemm_bf16(b, gsz, n, k, x, pk, scales, None, flags=flags)
        assert np.array_equal(y.view(np.uint32), expect.view(np.uint32)), flags


@pytest.mark.parametrize("b,g,zp", [(4, 128, True), (3, 32, True), (8, 128, False), (2, -1, True), (6, 32, False)])
def test_bf16_midbatch_kernel(b, g, zp):
    n, k, m = 304, 128 * 13, 77
    q, s16, z16 = o.make_layer(n, k, g, seed=70 + b, symmetric=not zp)
    s = o.round_to_bf16(s16.astype(np.float32))
    z = z16.astype(np.float32)
    x = o.round_to_bf16(o.make_activations(m, k, seed=9).astype(np.float32))
    pk = G.pack_device(q, b, True)
    ref = o.linear_f64(x, o.dequantize_bf16(q, s, z, b, g))
    for v in _mid_variants(b, g):
        y = _gemm_bf16(b, g, n, k, x, pk, s, z if zp else None, flags=3 | (v << 8))
        assert np.all(np.isfinite(y))
        assert np.max(np.abs(y - ref)) <= G.REL_TOL * np.max(np.abs(ref)), (b, g, zp, v)


@pytest.mark.parametrize("b", (2, 3, 4, 6, 8))
@pytest.mark.parametrize("zp", (True, False))
def test_bf16_prefill_weights_are_the_oracles_bit_for_bit(b, zp):
    # The prefill and mid-batch kernels multiply bf16 by bf16 on the matrix cores.  With the identity as
    # activations every output is one weight (plus exact zeros), so the result must be
    # dequantize() on bfloat16 tensors, bit for bit (integer zero points: one rounding on both
    # sides).  Ring tiles 128 x 256, 128 x 128, 128 x 192, the tail split, a staged tile, the three
    # tiles that split K inside the workgroup, the paired tiles, and three shapes of the mid-batch kernel.
    n, k, g = 304, 256, 128
    q, s16, z16 = o.make_layer(n, k, g, seed=300 + b, symmetric=not zp)
    s = o.round_to_bf16(s16.astype(np.float32))
    z = np.round(z16.astype(np.float32))
    x = np.eye(k, dtype=np.float32)
    pk = G.pack_device(q, b, True)
    w = o.dequantize_bf16(q, s, z, b, g)
    for cfg in (64, 67, 73, 72, 66, 74, 75, 76, 77, 89, 90, 80, 84, 88):
        y = _gemm_bf16(b, g, n, k, x, pk, s, z if zp else None, flags=3 | (cfg << 8))
        assert np.array_equal(y, w.T), (b, zp, cfg)


@pytest.mark.parametrize("flags", (3, 3 | (64 << 8), 3 | (65 << 8), 3 | (67 << 8), 3 | (72 << 8), 3 | (73 << 8), 3 | (74 << 8),
                                   3 | (75 << 8), 3 | (78 << 8), 3 | (79 << 8), 3 | (89 << 8), 3 | (90 << 8)))
def test_bf16_prefill_large_tiles(flags):
    # default choice for a large batch, and the ring, split, mixed and largest tiles forced
    n, k, m, b, g = 2048, 1024, 2048, 4, 128
    q, s16, z16 = o.make_layer(n, k, g, seed=77)
    s = o.round_to_bf16(s16.astype(np.float32))
    z = z16.astype(np.float32)
    x = o.round_to_bf16(o.make_activations(m, k, seed=8).astype(np.float32))
    pk = G.pack_device(q, b, True)
    y = _gemm_bf16(b, g, n, k, x, pk, s, z, flags=flags)
    rows = np.r_[0:64, m - 64:m]
    ref = o.linear_f64(x[rows], o.dequantize_bf16(q, s, z, b, g))
    assert np.all(np.isfinite(y))
    assert np.max(np.abs(y[rows] - ref)) <= G.REL_TOL * np.max(np.abs(ref))


@pytest.mark.parametrize("b,g,zp", [(4, 32, True), (8, 32, True), (3, -1, False), (6, 128, True), (2, 32, False), (8, -1, True)])
def test_bf16_64_row_split_tile_every_group_size(b, g, zp):
    # the 64 x 128 tile with K split in the workgroup on bf16 storage: ragged M and N, seven K tiles
    n, k, m = 304, 128 * 7, 200
    q, s16, z16 = o.make_layer(n, k, g, seed=50 + b, symmetric=not zp)
    s = o.round_to_bf16(s16.astype(np.float32))
    z = np.round(z16.astype(np.float32))
    x = o.round_to_bf16(o.make_activations(m, k, seed=b).astype(np.float32))
    pk = G.pack_device(q, b, True)
    y = _gemm_bf16(b, g, n, k, x, pk, s, z if zp else None, flags=3 | (89 << 8))
    ref = o.linear_f64(x, o.dequantize_bf16(q, s, z, b, g))
    assert np.all(np.isfinite(y))
    assert np.max(np.abs(y - ref)) <= G.REL_TOL * np.max(np.abs(ref))


@pytest.mark.parametrize("b,g,zp", [(4, 128, True), (3, 32, True), (8, 128, False), (2, -1, True), (6, 128, True)])
def test_prefill_tiles_agree_bit_for_bit(b, g, zp):
    # every tile accumulates the same products in the same order, so two tiles must give the same
    # bits; the ring tile (hand-counted waits, asynchronous copies into LDS) is compared with a
    # staged tile on a problem large enough to keep every CU busy for several rounds
    n, k, m = 4096, 2048, 2048
    rng = np.random.default_rng(b)
    packed = torch.from_numpy(rng.integers(-2 ** 31, 2 ** 31, _lib.load().matgptq_packed_words(b, n, k),
                                           dtype=np.int64).astype(np.int32)).to(G.DEV)
    groups = n * (1 if g == -1 else k // g)
    scales = torch.from_numpy((rng.random(groups) * 0.01 + 1e-3).astype(np.float16)).to(G.DEV)
    zeros = torch.from_numpy(rng.integers(0, 256, groups).astype(np.float16)).to(G.DEV) if zp else None
    x = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float16)).to(G.DEV)
    ring = [G.gemm(b, g, n, k, x, packed, scales, zeros, flags=1 | (64 << 8)).clone() for _ in range(3)]
    ring.append(G.gemm(b, g, n, k, x, packed, scales, zeros, flags=1 | (67 << 8)).clone())  # 128 x 128 ring tile
    ring.append(G.gemm(b, g, n, k, x, packed, scales, zeros, flags=1 | (73 << 8)).clone())  # 128 x 192 ring tile
    staged = G.gemm(b, g, n, k, x, packed, scales, zeros, flags=1 | (66 << 8))  # 64 x 256, staged
    torch.cuda.synchronize()
    assert torch.isfinite(staged.float()).all()
    for y in ring:
        assert torch.equal(y, staged)


@pytest.mark.parametrize("b,g,zp,n,k,m", [(4, 128, True, 10240, 512, 2048), (3, 32, False, 8192 + 304, 256, 2000),
                                          (8, -1, True, 4096 + 16, 384, 4096), (2, 128, False, 528, 128, 130)])
def test_prefill_tail_of_narrow_tiles(b, g, zp, n, k, m):
    # 128 x 256 tiles for the whole rounds of resident workgroups, 128 x 128 tiles for the rest of
    # the weight rows, in one launch: same products in the same order as the plain 128 x 256 tile
    # (first case: the shape split of a Llama-3-70B qkv layer at M = 2048; then ragged N and M, a
    # tail of a single row block, and a layer with no whole round at all)
    rng = np.random.default_rng(b)
    packed = torch.from_numpy(rng.integers(-2 ** 31, 2 ** 31, _lib.load().matgptq_packed_words(b, n, k),
                                           dtype=np.int64).astype(np.int32)).to(G.DEV)
    groups = n * (1 if g == -1 else k // g)
    scales = torch.from_numpy((rng.random(groups) * 0.01 + 1e-3).astype(np.float16)).to(G.DEV)
    zeros = torch.from_numpy(rng.integers(0, 256, groups).astype(np.float16)).to(G.DEV) if zp else None
    x = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float16)).to(G.DEV)
    plain = G.gemm(b, g, n, k, x, packed, scales, zeros, flags=1 | (64 << 8)).clone()
    tail = G.gemm(b, g, n, k, x, packed, scales, zeros, flags=1 | (72 << 8)).clone()
    torch.cuda.synchronize()
    assert torch.isfinite(plain.float()).all()
    assert torch.equal(tail, plain)
