"""The oracle against what pins it: closed forms, brute force, invariants, the C
restatement and the golden vectors produced by the reference's own functions
(src/quant_utils_matgpqt.py:9-22,202-224)."""
import numpy as np
import pytest

from oracle import c_oracle, matgptq_oracle as o

BITS = (2, 3, 4, 6, 8)
ALL = np.arange(256, dtype=np.uint8)


@pytest.mark.parametrize("b", BITS)
def test_slice_closed_form_all_codes(b):
    # independent closed form: round-half-up of q / 2^(8-b), saturated; identity at b = 8
    q = ALL.astype(np.int64)
    expect = q if b == 8 else np.minimum((q + (1 << (7 - b))) >> (8 - b), (1 << b) - 1)
    assert np.array_equal(o.slice_codes(ALL, b), expect.astype(np.uint8))


@pytest.mark.parametrize("b", BITS)
def test_slice_invariants(b):
    s = o.slice_codes(ALL, b).astype(int)
    assert np.all(np.diff(s) >= 0)                       # monotone
    assert s[255] == (1 << b) - 1                        # saturates at the top
    assert s.max() == (1 << b) - 1 and s.min() == 0
    if b < 8:
        zero_until = 1 << (7 - b)                        # s == 0  <=>  q < 2^(7-b)
        assert np.all(s[:zero_until] == 0) and np.all(s[zero_until:] > 0)
        # a b-bit slice depends on the top b+1 bits only
        low_mask = (1 << (7 - b)) - 1
        assert np.array_equal(o.slice_codes(ALL & ~np.uint8(low_mask), b), s.astype(np.uint8))
    else:
        assert np.array_equal(s, ALL)


def test_slice_master_equal_slice_is_floor():
    # the branch of src/quant_utils_matgpqt.py:13-14 (no rounding bit) for a 4-bit master
    q = ALL
    assert np.array_equal(o.slice_codes(q, 4, master_bits=4), np.minimum(q >> 4, 15))


@pytest.mark.parametrize("b", BITS)
def test_slice_matches_golden_and_c(b, golden):
    row = golden["slice_table"][BITS.index(b)]
    assert np.array_equal(o.slice_codes(ALL, b), row)
    assert np.array_equal(c_oracle.slice_codes(ALL, b), row)


@pytest.mark.parametrize("b", BITS)
def test_dequantize_matches_golden(b, golden):
    w = o.dequantize(golden["q"], golden["scale"], golden["zero"], b, 128)
    assert np.array_equal(w.view(np.uint16), golden[f"w_b{b}"].view(np.uint16))
    wc = c_oracle.dequantize(golden["q"], golden["scale"], golden["zero"], b, 128)
    assert np.array_equal(wc.view(np.uint16), golden[f"w_b{b}"].view(np.uint16))


def test_dequantize_other_group_sizes_match_golden(golden):
    for tag, g in (("g32", 32), ("gm1", -1)):
        w = o.dequantize(golden["q"], golden[f"scale_{tag}"], golden[f"zero_{tag}"], 3, g)
        assert np.array_equal(w.view(np.uint16), golden[f"w_b3_{tag}"].view(np.uint16))


@pytest.mark.parametrize("b", BITS)
def test_forward_matches_golden(b, golden):
    # the reference's CPU F.linear accumulates in its own order: compare to fp16 resolution
    y = o.fake_matryoshka_linear(golden["x"], golden["q"], golden["scale"], golden["zero"], b, 128)
    ref = golden[f"y_b{b}"].astype(np.float64)
    assert np.max(np.abs(y.astype(np.float64) - ref)) <= 2 ** -10 * np.max(np.abs(ref))
    yc = c_oracle.forward(golden["x"], golden["q"], golden["scale"], golden["zero"], b, 128)
    assert np.array_equal(yc.view(np.uint16), y.view(np.uint16))


@pytest.mark.parametrize("b", BITS)
@pytest.mark.parametrize("g", (128, 32, -1))
def test_dequantize_is_one_rounding_of_exact_value(b, g):
    # integers (c << (8-b)) - z are exact in fp16, so W must be the correctly rounded product
    q, s, z = o.make_layer(32, 256, g, seed=b)
    w = o.dequantize(q, s, z, b, g)
    gs = 256 if g == -1 else g
    shifted = o.slice_codes(q, b).astype(np.float64) * (1 << (8 - b))
    exact = np.repeat(s.astype(np.float64), gs, 1) * (shifted - np.repeat(z.astype(np.float64), gs, 1))
    assert np.array_equal(w.view(np.uint16), exact.astype(np.float16).view(np.uint16))


@pytest.mark.parametrize("b", BITS)
def test_symmetric_zero_reduces_to_kernel_form(b):
    # zero = 128 <=> (c - 2^(b-1)) * scale * 2^(8-b), the kernel test's formula
    # (inference_lib/test_matgptq_matmul.py:40); power-of-two factors commute with rounding
    q, s, _ = o.make_layer(16, 256, 128, seed=3)
    z = np.full_like(s, 128.0)
    a = o.dequantize(q, s, z, b, 128)
    k = o.dequantize_kernel_form(o.slice_codes(q, b), s, b, 128)
    assert np.array_equal(a.view(np.uint16), k.view(np.uint16))


@pytest.mark.parametrize("b", BITS)
def test_reference_test_regime_is_exact(b):
    # 0/1 scales and integer activations (inference_lib/test_matgptq_matmul.py:33-38):
    # every product and partial sum is an integer below 2^24, so any accumulation order
    # gives the same value and the fp16 result is unique
    rng = np.random.default_rng(1)
    n, k, m = 16, 1024, 8
    codes = rng.integers(0, 1 << b, (n, k), dtype=np.uint8)
    scales = rng.integers(0, 2, (n, k // 128)).astype(np.float16)
    x = np.round(rng.standard_normal((m, k))).astype(np.float16)
    w = o.dequantize_kernel_form(codes, scales, b, 128)
    y64 = o.linear_f64(x, w)
    assert np.array_equal(y64, np.round(y64))
    y32 = x.astype(np.float32) @ w.astype(np.float32).T
    assert np.array_equal(y32.astype(np.float64), y64)
    assert np.array_equal(o.linear(x, w).view(np.uint16), y64.astype(np.float16).view(np.uint16))


def test_c_oracle_half_conversion_is_round_to_nearest_even():
    lib = c_oracle.lib()
    rng = np.random.default_rng(0)
    v = np.concatenate([rng.standard_normal(20000) * 10.0 ** rng.integers(-9, 5, 20000),
                        [0.0, -0.0, 65504.0, 65519.9, 6.1e-5, 6.0e-8, 2.98e-8, 2049.0, 2051.0]])
    got = np.array([lib.matgptq_oracle_f64_to_f16(float(t)) for t in v], dtype=np.uint16)
    with np.errstate(over="ignore"):
        assert np.array_equal(got, v.astype(np.float16).view(np.uint16))


def test_c_oracle_matches_numpy_on_random_layer():
    q, s, z = o.make_layer(48, 384, 128, seed=5)
    x = o.make_activations(5, 384, seed=5, outlier_frac=0.01)
    for b in BITS:
        a = o.fake_matryoshka_linear(x, q, s, z, b, 128)
        c = c_oracle.forward(x, q, s, z, b, 128)
        assert np.array_equal(a.view(np.uint16), c.view(np.uint16))


# ---------------------------------------------------------------- bfloat16 forms

def test_bf16_rounding_matches_torch_exhaustively():
    import torch
    hi = np.arange(1 << 16, dtype=np.uint32) << 16
    for lo in (0x0000, 0x7FFF, 0x8000, 0x8001, 0xFFFF):
        a = (hi | lo).view(np.float32)
        mine = o.round_to_bf16(a)
        ref = torch.from_numpy(a.copy()).to(torch.bfloat16).float().numpy()
        nan = np.isnan(ref)
        assert np.array_equal(np.isnan(mine), nan)
        assert np.array_equal(mine[~nan].view(np.uint32), ref[~nan].view(np.uint32)), hex(lo)
    assert np.array_equal(o.bf16_from_bits(o.bf16_bits(mine[~nan])), mine[~nan])


@pytest.mark.parametrize("b", BITS)
def test_bf16_dequantize_and_forward_match_golden(b, golden):
    w = o.dequantize_bf16(golden["q"], golden["scale_bf16"], golden["zero_bf16"], b, 128)
    assert np.array_equal(w.view(np.uint32), golden[f"w_bf16_b{b}"].view(np.uint32))
    y = o.fake_matryoshka_linear_bf16(golden["x_bf16"], golden["q"], golden["scale_bf16"],
                                      golden["zero_bf16"], b, 128)
    ref = golden[f"y_bf16_b{b}"].astype(np.float64)
    # torch accumulates the bfloat16 product in fp32: within one bfloat16 step of the value
    assert np.max(np.abs(y - ref)) <= 2.0 ** -7 * np.max(np.abs(ref))


@pytest.mark.parametrize("b", BITS)
def test_bf16_torch_path_matches_golden(b, golden):
    import torch
    from oracle import torch_path
    q = torch.from_numpy(golden["q"])
    s = torch.from_numpy(golden["scale_bf16"]).to(torch.bfloat16)
    z = torch.from_numpy(golden["zero_bf16"]).to(torch.bfloat16)
    x = torch.from_numpy(golden["x_bf16"]).to(torch.bfloat16)
    w = torch_path.get_weight(q, s, z, 8, b)
    assert w.dtype == torch.bfloat16
    assert np.array_equal(w.float().numpy().view(np.uint32), golden[f"w_bf16_b{b}"].view(np.uint32))
    y = torch_path.forward(x, q, s, z, 8, b)
    assert np.array_equal(y.float().numpy().view(np.uint32), golden[f"y_bf16_b{b}"].view(np.uint32))
