"""The batch-1..4 kernel (gemv_gfx950.hip), and its instantiation for five to eight batch rows,
against the oracle, through the C ABI.

Every instantiation (tiles per wave and round x row blocks per workgroup), every bitwidth,
both zero-point forms, ragged row-block counts and ragged rounds of K tiles, both storage types,
the three group sizes.
"""
import numpy as np
import pytest
import torch

from matgptq_amd import _lib
from oracle import matgptq_oracle as o
from tests import _gpu_util as G

pytestmark = pytest.mark.gpu
BITS = (2, 3, 4, 6, 8)
SHAPES = range(7)  # (T, R) entries of the kernel: (8,1) (4,1) (4,2) (2,2) (2,4) (2,1) (4,4)


def gemv_flags(shape, waves=0, base=1):
    return base | ((100 + shape) << 8) | (waves << 18)


@pytest.mark.parametrize("zp", (False, True))
@pytest.mark.parametrize("b", BITS)
def test_gemv_every_instantiation(b, zp):
    # 5 row blocks (ragged for two and four row blocks per workgroup), 13 K tiles (the last
    # round of every shape is ragged; with two tiles per wave some waves have no tile at all)
    n, k = 80, 128 * 13
    lay = G.Layer(n, k, b, 128, seed=40 + b, zero_points=zp)
    for m in (1, 2, 3, 4):
        x = o.make_activations(m, k, seed=m + b)
        G.assert_close_to_oracle(lay.run(x), x, lay.w, f"default b={b} zp={zp} M={m}")
        assert _lib.describe_plan(b, 128, n, k, m, zp).startswith("gemv")
        for shape in SHAPES:
            for waves in (0, 1, 3, 16):
                y = lay.run(x, flags=gemv_flags(shape, waves))
                G.assert_close_to_oracle(y, x, lay.w, f"b={b} zp={zp} M={m} shape={shape} W={waves}")
                G.assert_regression_bound(y, x, lay.w, f"b={b} zp={zp} M={m} shape={shape} W={waves}")


@pytest.mark.parametrize("g", (32, -1))
@pytest.mark.parametrize("zp", (False, True))
@pytest.mark.parametrize("b", BITS)
def test_gemv_group_sizes_32_and_per_row(b, zp, g):
    # a scale per octet of a tile (the row groups of the activation operand take turns per octet)
    # and a scale per weight row; ragged row blocks and rounds as above
    n, k = 80, 128 * 13
    lay = G.Layer(n, k, b, g, seed=60 + b, zero_points=zp)
    for m in (1, 2, 3, 4):
        x = o.make_activations(m, k, seed=m + b, outlier_frac=0.01)
        assert _lib.describe_plan(b, g, n, k, m, zp).startswith("gemv")
        G.assert_close_to_oracle(lay.run(x), x, lay.w, f"default b={b} g={g} zp={zp} M={m}")
        for shape in (1, 2):
            for waves in (0, 1, 3, 16):
                y = lay.run(x, flags=gemv_flags(shape, waves))
                G.assert_close_to_oracle(y, x, lay.w, f"b={b} g={g} zp={zp} M={m} shape={shape} W={waves}")
                G.assert_regression_bound(y, x, lay.w, f"b={b} g={g} zp={zp} M={m} shape={shape} W={waves}")


@pytest.mark.parametrize("g", (32, -1))
def test_gemv_group_sizes_exact_in_the_reference_test_regime(g):
    # 0/1 scales, integer activations, symmetric form: the closed form, bit for bit
    rng = np.random.default_rng(6)
    n, k = 48, 4096
    G_ = 1 if g == -1 else k // g
    for b in BITS:
        codes = rng.integers(0, 1 << b, (n, k), dtype=np.uint8)
        scales = np.round(rng.random((n, G_))).astype(np.float16)
        if g == -1:
            scales[:] = 1.0  # (a row of 4096 columns at scale 0 would test nothing)
        pk = G.pack_device(codes, b, from_master=False)
        sd = G.reorder_device(scales, n, k, g)
        w = o.dequantize_kernel_form(codes, scales, b, g)
        for m in (1, 4):
            x = np.round(rng.standard_normal((m, k))).astype(np.float16)
            expect = o.linear_f64(x, w).astype(np.float16)
            for shape in (1, 2):
                y = G.gemm(b, g, n, k, G.to_dev(x), pk, sd, None, flags=gemv_flags(shape)).cpu().numpy()
                assert np.array_equal(y.view(np.uint16), expect.view(np.uint16)), (b, g, m, shape)


def test_gemv_group_sizes_agree_with_the_decode_kernel():
    n, k, b = 1024, 4096, 4
    for g in (32, -1):
        lay = G.Layer(n, k, b, g, seed=11)
        for m in (1, 3):
            x = o.make_activations(m, k, seed=m)
            a = lay.run(x).astype(np.float64)
            c = lay.run(x, flags=1 | (1 << 16)).astype(np.float64)  # burst flavour: the decode kernel
            assert _lib.describe_plan(b, g, n, k, m, True, 1 | (1 << 16)).startswith("decode")
            assert np.max(np.abs(a - c)) <= 2.0 ** -9 * np.max(np.abs(c))


@pytest.mark.parametrize("g", (128, -1))
@pytest.mark.parametrize("zp", (False, True))
@pytest.mark.parametrize("b", BITS)
def test_gemv_five_to_eight_batch_rows(b, zp, g):
    # two tiles x eight batch rows in the activation operand, the sums of a tile through a table in
    # LDS; 5 row blocks and 13 K tiles as above (ragged for two row blocks per workgroup, ragged rounds,
    # an odd number of tiles: the last chain of MFMAs covers one tile)
    n, k = 80, 128 * 13
    lay = G.Layer(n, k, b, g, seed=40 + b, zero_points=zp)
    for m in (5, 6, 7, 8):
        x = o.make_activations(m, k, seed=m + b, outlier_frac=0.01)
        assert _lib.describe_plan(b, g, n, k, m, zp).startswith("gemv")
        G.assert_close_to_oracle(lay.run(x), x, lay.w, f"default b={b} g={g} zp={zp} M={m}")
        for shape in (1, 2):
            for waves in (0, 1, 3, 16):
                if shape == 2 and waves == 16:  # more LDS than a CU has
                    with pytest.raises(_lib.MatGPTQError, match="variant"):
                        lay.run(x, flags=gemv_flags(shape, waves))
                    continue
                y = lay.run(x, flags=gemv_flags(shape, waves))
                G.assert_close_to_oracle(y, x, lay.w, f"b={b} g={g} zp={zp} M={m} shape={shape} W={waves}")
                G.assert_regression_bound(y, x, lay.w, f"b={b} g={g} zp={zp} M={m} shape={shape} W={waves}")


def test_gemv_five_to_eight_batch_rows_long_k():
    # 224 K tiles: several rounds per wave, fifteen waves with two row blocks per workgroup (LDS)
    lay = G.Layer(64, 28672, 4, 128, seed=4)
    x = o.make_activations(8, 28672, seed=8)
    assert _lib.describe_plan(4, 128, 64, 28672, 8, True, gemv_flags(2)) == "gemv b4 g128 zp1 T4 R2 W15 pad0"
    for shape in (1, 2):
        y = lay.run(x, flags=gemv_flags(shape))
        G.assert_close_to_oracle(y, x, lay.w, f"long K shape={shape}")
        G.assert_regression_bound(y, x, lay.w, f"long K shape={shape}")


def test_gemv_five_to_eight_batch_rows_exact_in_the_reference_test_regime():
    rng = np.random.default_rng(5)
    n, k = 48, 4096
    for b in BITS:
        codes = rng.integers(0, 1 << b, (n, k), dtype=np.uint8)
        scales = np.round(rng.random((n, k // 128))).astype(np.float16)
        pk = G.pack_device(codes, b, from_master=False)
        sd = G.reorder_device(scales, n, k, 128)
        w = o.dequantize_kernel_form(codes, scales, b, 128)
        for m in (5, 8):
            x = np.round(rng.standard_normal((m, k))).astype(np.float16)
            expect = o.linear_f64(x, w).astype(np.float16)
            for shape in (1, 2):
                y = G.gemm(b, 128, n, k, G.to_dev(x), pk, sd, None, flags=gemv_flags(shape)).cpu().numpy()
                assert np.array_equal(y.view(np.uint16), expect.view(np.uint16)), (b, m, shape)


def test_gemv_is_not_taken_outside_its_domain():
    assert _lib.describe_plan(4, 128, 4096, 4096, 9, True).split()[0] in ("decode-burst", "midbatch")
    assert _lib.describe_plan(4, 128, 28672, 4096, 5, True).split()[0] in ("decode-burst", "midbatch")
    assert _lib.describe_plan(4, 32, 4096, 4096, 5, True).split()[0].startswith(("decode", "midbatch"))
    with pytest.raises(_lib.MatGPTQError, match="variant"):  # group 32: shapes 1 and 2 only
        G.Layer(32, 256, 4, 32, seed=1).run(o.make_activations(1, 256, seed=1), flags=gemv_flags(0))
    with pytest.raises(_lib.MatGPTQError, match="variant"):
        G.Layer(32, 256, 4, 128, seed=1).run(o.make_activations(5, 256, seed=1), flags=gemv_flags(0))
    with pytest.raises(_lib.MatGPTQError, match="variant"):
        G.Layer(32, 256, 4, 128, seed=1).run(o.make_activations(1, 256, seed=1), flags=gemv_flags(7))


@pytest.mark.parametrize("b", (2, 4, 8))
def test_gemv_long_k_several_rounds(b):
    # 224 K tiles (the Llama-3-70B down projection): 16 waves walk 3.5 rounds of four tiles
    n, k = 64, 28672
    lay = G.Layer(n, k, b, 128, seed=b)
    for m in (1, 4):
        x = o.make_activations(m, k, seed=m)
        y = lay.run(x)
        G.assert_close_to_oracle(y, x, lay.w, f"long K b={b} M={m}")
        G.assert_regression_bound(y, x, lay.w, f"long K b={b} M={m}")
    assert _lib.describe_plan(b, 128, n, k, 1, True) == f"gemv b{b} g128 zp1 T4 R1 W16 pad0"


def test_gemv_exact_in_the_reference_test_regime():
    # 0/1 scales, integer activations, symmetric form: every product and partial sum is an
    # integer below 2^24, so the output must equal the closed form bit for bit
    # (inference_lib/test_matgptq_matmul.py:29-49)
    rng = np.random.default_rng(5)
    n, k = 48, 4096
    for b in BITS:
        codes = rng.integers(0, 1 << b, (n, k), dtype=np.uint8)
        scales = np.round(rng.random((n, k // 128))).astype(np.float16)
        pk = G.pack_device(codes, b, from_master=False)
        sd = G.reorder_device(scales, n, k, 128)
        w = o.dequantize_kernel_form(codes, scales, b, 128)
        for m in (1, 2, 4):
            x = np.round(rng.standard_normal((m, k))).astype(np.float16)
            expect = o.linear_f64(x, w).astype(np.float16)
            for shape in SHAPES:
                y = G.gemm(b, 128, n, k, G.to_dev(x), pk, sd, None, flags=gemv_flags(shape)).cpu().numpy()
                assert np.array_equal(y.view(np.uint16), expect.view(np.uint16)), (b, m, shape)


def test_gemv_outlier_channels():
    lay = G.Layer(256, 4096, 3, 128, seed=12)
    for m in (1, 2, 4):
        x = o.make_activations(m, 4096, seed=3, outlier_frac=0.01, outlier_gain=20.0)
        for shape in SHAPES:
            G.assert_close_to_oracle(lay.run(x, flags=gemv_flags(shape)), x, lay.w, f"outliers M={m} shape={shape}")


def test_gemv_agrees_with_the_decode_kernel():
    # same products, another summation order: agreement to fp32 rounding of the accumulation
    n, k, b = 1024, 4096, 4
    lay = G.Layer(n, k, b, 128, seed=9)
    for m in (1, 3):
        x = o.make_activations(m, k, seed=m)
        a = lay.run(x).astype(np.float64)
        c = lay.run(x, flags=1 | (1 << 16)).astype(np.float64)  # burst flavour: the decode kernel
        assert _lib.describe_plan(b, 128, n, k, m, True, 1 | (1 << 16)).startswith("decode")
        assert np.max(np.abs(a - c)) <= 2.0 ** -9 * np.max(np.abs(c))


def test_gemv_output_does_not_depend_on_earlier_calls():
    # the kernel keeps its staged activations in LDS only: two layers, alternating, same bits
    la, lb = G.Layer(96, 1024, 4, 128, seed=1), G.Layer(96, 1024, 4, 128, seed=2)
    x = o.make_activations(1, 1024, seed=1)
    ya, yb = la.run(x), lb.run(x)
    for _ in range(3):
        assert np.array_equal(la.run(x), ya)
        assert np.array_equal(lb.run(x), yb)


@pytest.mark.parametrize("b", BITS)
def test_gemv_bf16_storage(b):
    n, k = 80, 128 * 13
    q, s16, z16 = o.make_layer(n, k, 128, seed=3 * b)
    s = o.round_to_bf16(s16.astype(np.float32))
    z = z16.astype(np.float32)
    pk = G.pack_device(q, b, True)
    L = G.lib()

    def dev_bf16(a):
        return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16).to(G.DEV)

    def reorder(a):
        src = dev_bf16(a)
        out = torch.empty_like(src)
        _lib.check(L.matgptq_reorder_scales_device(src.data_ptr(), n, k, 128, out.data_ptr(), G.stream()))
        return out

    sr, zr = reorder(s), reorder(z)
    for m in (1, 4, 7):
        x = o.round_to_bf16(o.make_activations(m, k, seed=m + b, outlier_frac=0.01).astype(np.float32))
        xd = dev_bf16(x)
        for zeros, zz in ((zr, z), (None, np.full_like(z, 128.0))):
            ref = o.linear_f64(x, o.dequantize_bf16(q, s, zz, b, 128))
            for shape in (1, 2, 4) if m <= 4 else (1, 2):
                y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=G.DEV)
                _lib.check(L.matgptq_gemm(b, 128, n, k, m, pk.data_ptr(), sr.data_ptr(),
                                          zeros.data_ptr() if zeros is not None else None, xd.data_ptr(),
                                          y.data_ptr(), G.stream(), gemv_flags(shape, base=3)))
                torch.cuda.synchronize()
                yv = y.float().cpu().numpy()
                assert np.all(np.isfinite(yv))
                assert np.max(np.abs(yv - ref)) <= G.REL_TOL * np.max(np.abs(ref)), (b, m, shape)
                assert np.array_equal(o.round_to_bf16(yv), yv)
