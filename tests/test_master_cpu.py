"""Master-resident bit planes on the host: the in-register slice the GEMM kernels run (the same
source, matgptq_amd/csrc/master_layout.h, compiled for the host) against the golden slice table the
reference's matryoshka_slice produced, and the layout's structure.  No GPU work."""
import numpy as np
import pytest
from hypothesis import given, settings, strategies as st

from matgptq_amd import _lib
from oracle import matgptq_oracle as o

BITS = (2, 3, 4, 6, 8)


def L():
    return _lib.load()


def pack_master(codes):
    n, k = codes.shape
    out = np.zeros(L().matgptq_master_words(n, k), dtype=np.uint32)
    _lib.check(L().matgptq_pack_master_host(codes.ctypes.data, n, k, out.ctypes.data))
    return out


def unpack_master(planes, n, k, b):
    out = np.full((n, k), 0xAA, dtype=np.uint8)
    _lib.check(L().matgptq_unpack_master_host(planes.ctypes.data, n, k, b, out.ctypes.data))
    return out


def test_size_is_one_byte_per_weight():
    assert L().matgptq_master_words(16, 128) == 16 * 128 // 4
    assert L().matgptq_master_words(28672, 4096) == 28672 * 4096 // 4
    assert L().matgptq_master_words(15, 128) == 0 and L().matgptq_master_words(16, 100) == 0


@pytest.mark.parametrize("b", BITS)
def test_slice_from_planes_equals_the_reference_slice_table(b, golden):
    # every master code at every position of a lane (octet, element), in every k-quarter and row
    table = golden["slice_table"][BITS.index(b)]
    n, k = 16, 128 * 16
    codes = (np.arange(n * k, dtype=np.int64).reshape(n, k) * 7 + np.arange(n)[:, None] * 31) % 256
    codes = codes.astype(np.uint8)
    for shift in range(0, 256, 37):  # each position sees many different codes
        c = ((codes.astype(np.int64) + shift) % 256).astype(np.uint8)
        got = unpack_master(pack_master(c), n, k, b)
        assert np.array_equal(got, table[c]), (b, shift)
    assert np.array_equal(table, o.slice_codes(np.arange(256, dtype=np.uint8), b))


@pytest.mark.parametrize("b", BITS)
def test_saturation_and_rounding_neighbours(b):
    # tiles of nothing but the codes around every rounding threshold and the saturating top
    n, k = 16, 128
    for q in (0, 1, (1 << (7 - b)) - 1 if b < 8 else 0, 1 << (7 - b) if b < 8 else 1, 127, 128, 254, 255,
              256 - (1 << (8 - b)), 255 - (1 << (7 - b)) if b < 8 else 255):
        c = np.full((n, k), q, dtype=np.uint8)
        assert np.array_equal(unpack_master(pack_master(c), n, k, b), o.slice_codes(c, b)), (b, q)
    # a checkerboard of saturating and non-saturating neighbours: no carry between fields
    c = np.where((np.arange(n)[:, None] + np.arange(k)[None, :]) % 2 == 0, 255, 0).astype(np.uint8)
    assert np.array_equal(unpack_master(pack_master(c), n, k, b), o.slice_codes(c, b))


@settings(max_examples=25, deadline=None)
@given(b=st.sampled_from(BITS), nb=st.integers(1, 3), kb=st.integers(1, 3), seed=st.integers(0, 2 ** 31 - 1))
def test_slice_from_planes_property(b, nb, kb, seed):
    rng = np.random.default_rng(seed)
    n, k = 16 * nb, 128 * kb
    c = rng.integers(0, 256, (n, k), dtype=np.uint8)
    assert np.array_equal(unpack_master(pack_master(c), n, k, b), o.slice_codes(c, b))


def test_a_bitwidth_reads_only_its_prefix_of_the_tile():
    # words beyond the segments a bitwidth reads must not influence its slice: flip them
    rng = np.random.default_rng(3)
    n, k = 16, 256
    c = rng.integers(0, 256, (n, k), dtype=np.uint8)
    planes = pack_master(c).reshape(-1, 512)  # one row per tile
    # tile words: S0 = [0, 192), S1 = [192, 256), S2 = [256, 320), S3 = [320, 512)
    prefix = {2: 192, 3: 256, 4: 320, 6: 512, 8: 512}
    for b in BITS:
        noisy = planes.copy()
        noisy[:, prefix[b]:] ^= 0xFFFFFFFF
        assert np.array_equal(unpack_master(noisy.reshape(-1), n, k, b), o.slice_codes(c, b)), b
        if prefix[b] > 0:
            broken = planes.copy()
            broken[:, :prefix[b]] ^= 0xFFFFFFFF
            assert not np.array_equal(unpack_master(broken.reshape(-1), n, k, b), o.slice_codes(c, b))


def test_planes_hold_the_bits_most_significant_first():
    # a code with only bit p set shows up in exactly the plane of that bit
    n, k = 16, 128
    segments = {7: (0, 192), 6: (0, 192), 5: (0, 192), 4: (192, 256), 3: (256, 320), 2: (320, 512), 1: (320, 512), 0: (320, 512)}
    for p in range(8):
        planes = pack_master(np.full((n, k), 1 << p, dtype=np.uint8))
        lo, hi = segments[p]
        assert planes[lo:hi].any()
        rest = np.concatenate([planes[:lo], planes[hi:]])
        assert not rest.any(), p
        assert int(sum(bin(int(w)).count("1") for w in planes)) == n * k


def test_error_codes():
    lib = L()
    assert lib.matgptq_pack_master_host(None, 16, 128, None) == -4
    assert lib.matgptq_pack_master_host(1, 15, 128, 1) == -3
    assert lib.matgptq_unpack_master_host(1, 16, 128, 5, 1) == -1
    assert lib.matgptq_gemm_master(4, 128, 16, 128, 1, None, 1, None, 1, 1, None, 0, None, 1) == -4
    # the batch-1..4 kernel and the mid-batch kernel read the planes themselves; outside them a
    # workspace is needed
    assert lib.matgptq_gemm_master_workspace_bytes(4, 128, 4096, 4096, 1, 1) == 0
    assert lib.matgptq_gemm_master_workspace_bytes(4, 128, 4096, 4096, 4, 1) == 0
    assert lib.matgptq_gemm_master_workspace_bytes(4, 128, 4096, 4096, 5, 1) == 0
    assert lib.matgptq_gemm_master_workspace_bytes(3, 32, 4096, 4096, 1, 1) == 0
    assert lib.matgptq_gemm_master_workspace_bytes(3, 32, 4096, 4096, 7, 1) == 0
    assert lib.matgptq_gemm_master_workspace_bytes(4, 128, 4096, 4096, 64, 1) == 0
    # (up to 128 batch rows a shape whose own plan is another kernel takes the mid-batch kernel here)
    assert lib.matgptq_gemm_master_workspace_bytes(8, 128, 28672, 4096, 8, 1) == 0
    assert lib.matgptq_gemm_master_workspace_bytes(4, 128, 28672, 4096, 128, 1) == 0
    assert lib.matgptq_gemm_master_workspace_bytes(4, 128, 28672, 4096, 129, 1) == 28672 * 4096 // 2
    assert lib.matgptq_gemm_master_workspace_bytes(8, 128, 28672, 4096, 8, 1 | (1 << 16)) == 28672 * 4096   # decode kernel asked for
    assert lib.matgptq_gemm_master_workspace_bytes(4, 128, 4096, 4096, 2048, 1) == 4096 * 4096 // 2
    assert lib.matgptq_gemm_master(4, 128, 4096, 4096, 2048, 1, 1, None, 1, 1, None, 0, None, 1) == -9
    assert lib.matgptq_gemm_master(4, 128, 4096, 4096, 2048, 1, 1, None, 1, 1, 1, 100, None, 1) == -9
    assert "workspace" in lib.matgptq_strerror(-9).decode()


def test_batches_of_one_to_four_rows_never_need_a_workspace():
    """Whatever gemv shape the planner prefers on pre-sliced codes (four row blocks per workgroup at
    2 and 3 bits on layers with many rows has no instantiation on planes), a call on planes with one
    to four batch rows reads them in the kernel."""
    lib = L()
    for bits in (2, 3, 4, 6, 8):
        for g in (128, 32, -1):
            for n, k in ((4096, 4096), (6144, 4096), (28672, 4096), (4096, 14336), (57344, 8192), (128256, 4096)):
                if bits * n * k // 8 >= 1 << 32 or n * k >= 1 << 32:
                    continue
                for m in (1, 2, 3, 4):
                    assert lib.matgptq_gemm_master_workspace_bytes(bits, g, n, k, m, 1) == 0, (bits, g, n, k, m)
    # the case that used to fall back to slicing 44 MB per call
    assert lib.matgptq_gemm_master_workspace_bytes(3, 128, 28672, 4096, 3, 0) == 0


def test_workspace_size_covers_the_call_with_and_without_zero_points():
    """The planner's choice can depend on whether zero points are passed; the size covers both.
    b = 2, g = 32, 18128 x 31872 at M = 182: mid-batch kernel with zero points, the 128 x 256 tile
    split over eight waves (which needs the sliced tensor) without."""
    lib = L()
    bits, g, n, k, m = 2, 32, 18128, 31872, 182
    need = lib.matgptq_gemm_master_workspace_bytes(bits, g, n, k, m, 1)
    assert need == bits * n * k // 8
    described = {zp: _describe(lib, bits, g, n, k, m, zp) for zp in (0, 1)}
    assert described[1].startswith("midbatch") and described[0].startswith("prefill"), described


def _describe(lib, bits, g, n, k, m, zp, flags=1):
    import ctypes
    buf = ctypes.create_string_buffer(128)
    assert lib.matgptq_describe_plan(bits, g, n, k, m, zp, flags, buf, 128) == 0
    return buf.value.decode()
