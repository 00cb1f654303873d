"""C ABI on the host: every declared symbol is exported, the packers round-trip, the
size contract of the reference's op holds, errors come back as codes.  No GPU work."""
import ctypes
import os
import re

import numpy as np
import pytest
from hypothesis import given, settings, strategies as st

from matgptq_amd import _lib
from oracle import matgptq_oracle as o

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BITS = (2, 3, 4, 6, 8)


def L():
    return _lib.load()


def test_every_declared_symbol_is_exported():
    header = open(os.path.join(ROOT, "include", "matgptq_abi.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    names = set(re.findall(r"\b(matgptq_[a-z_0-9]+)\s*\(", header))
    assert names == set(_lib.EXPORTS)
    lib = ctypes.CDLL(_lib.ABI_PATH)
    for n in sorted(names):
        assert hasattr(lib, n), n
    assert L().matgptq_abi_version() == 2


@pytest.mark.parametrize("b", BITS)
def test_packed_size_contract(b):
    # bitwidth * N * K / 32 words (inference_lib/matgptq_cuda/csrc/bindings.cpp:68,160)
    for n, k in ((16, 128), (4096, 4096), (28672, 4096)):
        assert L().matgptq_packed_words(b, n, k) == b * n * k // 32
    assert L().matgptq_packed_words(5, 16, 128) == 0


def _pack(codes, b, slice_=0):
    n, k = codes.shape
    out = np.zeros(L().matgptq_packed_words(b, n, k), dtype=np.uint32)
    _lib.check(L().matgptq_pack_host(codes.ctypes.data, n, k, b, slice_, out.ctypes.data))
    return out


def _unpack(packed, n, k, b):
    out = np.zeros((n, k), dtype=np.uint8)
    _lib.check(L().matgptq_unpack_host(packed.ctypes.data, n, k, b, out.ctypes.data))
    return out


@pytest.mark.parametrize("b", BITS)
def test_pack_unpack_identity(b):
    rng = np.random.default_rng(b)
    for n, k in ((16, 128), (48, 384), (64, 1024)):
        c = rng.integers(0, 1 << b, (n, k), dtype=np.uint8)
        assert np.array_equal(_unpack(_pack(c, b), n, k, b), c)


@pytest.mark.parametrize("b", BITS)
def test_pack_every_position_is_independent(b):
    # a single non-zero code anywhere in a tile comes back alone: catches overlapping fields
    top = (1 << b) - 1
    for pos in range(0, 16 * 128, 37):
        c = np.zeros((16, 128), dtype=np.uint8)
        c[pos // 128, pos % 128] = top
        assert np.array_equal(_unpack(_pack(c, b), 16, 128, b), c)


@settings(max_examples=30, deadline=None)
@given(st.sampled_from(BITS), st.integers(1, 3), st.integers(1, 3), st.integers(0, 2 ** 31 - 1))
def test_pack_unpack_identity_property(b, nb, kb, seed):
    rng = np.random.default_rng(seed)
    c = rng.integers(0, 1 << b, (16 * nb, 128 * kb), dtype=np.uint8)
    assert np.array_equal(_unpack(_pack(c, b), 16 * nb, 128 * kb, b), c)


@pytest.mark.parametrize("b", BITS)
def test_pack_from_master_slices_like_the_oracle(b):
    rng = np.random.default_rng(100 + b)
    q = rng.integers(0, 256, (32, 256), dtype=np.uint8)
    assert np.array_equal(_unpack(_pack(q, b, 1), 32, 256, b), o.slice_codes(q, b))
    # all 256 master codes in one tile
    q = np.tile(np.arange(256, dtype=np.uint8), 8).reshape(16, 128)
    assert np.array_equal(_unpack(_pack(q, b, 1), 16, 128, b), o.slice_codes(q, b))


@pytest.mark.parametrize("b", BITS)
def test_pack_unpack_identity_with_a_tail_of_64_columns(b):
    # K = 128 t + 64: tiles first, then the last 64 columns of every row as a bitstream; the size
    # stays bitwidth * N * K / 32 words
    rng = np.random.default_rng(20 + b)
    for n, k in ((16, 192), (48, 128 * 3 + 64)):
        c = rng.integers(0, 1 << b, (n, k), dtype=np.uint8)
        packed = _pack(c, b)
        assert packed.size == b * n * k // 32
        assert np.array_equal(_unpack(packed, n, k, b), c)
        q = rng.integers(0, 256, (n, k), dtype=np.uint8)
        assert np.array_equal(_unpack(_pack(q, b, 1), n, k, b), o.slice_codes(q, b))
    # the tail of a row is a plain little-endian bitstream: code j at bit j * b
    c = np.zeros((16, 192), dtype=np.uint8)
    c[5, 128 + 7] = (1 << b) - 1
    words = _pack(c, b)[64 * b:].reshape(16, 2 * b)  # behind the one tile of 64 b words
    bits = np.unpackbits(words[5].view(np.uint8), bitorder="little")
    assert bits.sum() == b and np.all(bits[7 * b:8 * b] == 1)
    assert not words[np.arange(16) != 5].any()


def test_pack_ignores_bits_above_the_bitwidth():
    rng = np.random.default_rng(9)
    c = rng.integers(0, 256, (16, 128), dtype=np.uint8)
    for b in (2, 3, 4, 6):
        assert np.array_equal(_unpack(_pack(c, b), 16, 128, b), c & ((1 << b) - 1))


@pytest.mark.parametrize("g", (128, 32, -1))
def test_reorder_scales_is_the_tile_transpose(g):
    n, k = 48, 512
    G = 1 if g == -1 else k // g
    s = np.arange(n * G, dtype=np.uint16).reshape(n, G)
    out = np.zeros_like(s)
    _lib.check(L().matgptq_reorder_scales_host(s.ctypes.data, n, k, g, out.ctypes.data))
    expect = s.reshape(n // 16, 16, G).transpose(0, 2, 1)
    assert np.array_equal(out.reshape(n // 16, G, 16), expect)


def test_error_codes():
    buf = np.zeros(16 * 128, dtype=np.uint8)
    out = np.zeros(8 * 16 * 128 // 32, dtype=np.uint32)
    lib = L()
    assert lib.matgptq_pack_host(buf.ctypes.data, 16, 128, 5, 0, out.ctypes.data) == -1
    assert lib.matgptq_pack_host(buf.ctypes.data, 15, 128, 4, 0, out.ctypes.data) == -3
    assert lib.matgptq_pack_host(buf.ctypes.data, 16, 64, 4, 0, out.ctypes.data) == -3
    assert lib.matgptq_pack_host(None, 16, 128, 4, 0, out.ctypes.data) == -4
    assert lib.matgptq_reorder_scales_host(buf.ctypes.data, 16, 128, 64, out.ctypes.data) == -2
    # argument checks of the GEMM come before any device work
    assert lib.matgptq_gemm(4, 128, 16, 128, 1, None, None, None, None, None, None, 1) == -4
    assert lib.matgptq_gemm(7, 128, 16, 128, 1, 1, 1, None, 1, 1, None, 1) == -1
    assert lib.matgptq_gemm(4, 48, 16, 128, 1, 1, 1, None, 1, 1, None, 1) == -2
    assert lib.matgptq_gemm(4, 128, 16, 128, 0, 1, 1, None, 1, 1, None, 1) == -8
    # 32-bit byte offsets inside the kernels: a packed tensor of 4 GiB or more is refused, and so is
    # a dimension above 2^24 (no device work: the pointers are never touched)
    assert lib.matgptq_gemm(8, 128, 65536, 65536, 1, 1, 1, None, 1, 1, None, 1) == -8
    assert lib.matgptq_gemm(4, 128, 65536, 131072, 1, 1, 1, None, 1, 1, None, 1) == -8
    assert lib.matgptq_gemm(2, 128, 16, 128, (1 << 24) + 1, 1, 1, None, 1, 1, None, 1) == -8
    assert lib.matgptq_gemm(2, 128, 16, 1 << 25, 1, 1, 1, None, 1, 1, None, 1) == -8
    assert lib.matgptq_gemm_master(2, 128, 65536, 65536, 1, 1, 1, None, 1, 1, None, 0, None, 1) == -8
    for code in range(-10, 1):
        assert lib.matgptq_strerror(code) != b"unknown error"
    with pytest.raises(_lib.MatGPTQError, match="bitwidth must be one of"):
        _lib.check(-1)


def test_describe_plan_regimes():
    # batch 1..4: the gemv kernel; five rows on: decode / mid-batch, or the gemv kernel again (below)
    assert _lib.describe_plan(4, 128, 4096, 4096, 1) == "gemv b4 g128 zp0 T4 R1 W8 pad0"
    assert _lib.describe_plan(4, 128, 4096, 14336, 1, True) == "gemv b4 g128 zp1 T4 R1 W16 pad0"
    assert _lib.describe_plan(4, 128, 4096, 4096, 4, True) == "gemv b4 g128 zp1 T4 R1 W8 pad0"
    assert _lib.describe_plan(4, 128, 28672, 4096, 4, True) == "gemv b4 g128 zp1 T4 R2 W8 pad0"
    assert _lib.describe_plan(4, 128, 4096, 4096, 1, True, 1 | (1 << 16)).startswith("decode-burst")
    assert _lib.describe_plan(4, 32, 4096, 4096, 1) == "gemv b4 g32 zp0 T4 R1 W8 pad0"
    assert _lib.describe_plan(4, -1, 4096, 4096, 4) == "gemv b4 g-1 zp0 T4 R1 W8 pad0"
    assert _lib.describe_plan(2, 128, 28672, 4096, 1, True) == "gemv b2 g128 zp1 T4 R2 W8 pad0"
    assert _lib.describe_plan(3, 128, 28672, 4096, 4, True) == "gemv b3 g128 zp1 T4 R4 W8 pad0"
    assert _lib.describe_plan(3, 128, 6144, 4096, 4, True) == "gemv b3 g128 zp1 T4 R2 W8 pad0"
    # two batch rows stage two rows (three and four stage four): one row block per workgroup stays ahead,
    # except for 2-bit tiles on layers with many rows
    assert _lib.describe_plan(4, 128, 28672, 4096, 2, True) == "gemv b4 g128 zp1 T4 R1 W8 pad0"
    assert _lib.describe_plan(3, 128, 28672, 4096, 2, True) == "gemv b3 g128 zp1 T4 R1 W8 pad0"
    assert _lib.describe_plan(2, 128, 28672, 4096, 2, True) == "gemv b2 g128 zp1 T4 R2 W8 pad0"
    assert _lib.describe_plan(4, 128, 28672, 4096, 3, True) == "gemv b4 g128 zp1 T4 R2 W8 pad0"
    assert _lib.describe_plan(4, 32, 4096, 4096, 5).startswith(("decode", "midbatch"))
    # five to sixteen rows: the mid-batch kernel, except at 8 bits on fp16 storage with one scale per
    # tile or row, on layers with many rows (two row blocks per workgroup only)
    assert _lib.describe_plan(4, 32, 28672, 4096, 8, True) == "midbatch b4 g32 zp1 R2 mb1"
    assert _lib.describe_plan(4, 32, 28672, 4096, 5, True) == "midbatch b4 g32 zp1 R2 mb1"
    assert _lib.describe_plan(8, 32, 28672, 4096, 8, True) == "midbatch b8 g32 zp1 R2 mb1"
    assert _lib.describe_plan(6, 32, 28672, 4096, 16, True) == "midbatch b6 g32 zp1 R2 mb1"
    assert _lib.describe_plan(8, 128, 28672, 4096, 8, True, 3) == "midbatch b8 g128 zp1 R2 mb1"  # bf16
    assert _lib.describe_plan(8, 128, 28672, 4096, 5, True).startswith("decode")
    assert _lib.describe_plan(8, -1, 28672, 4096, 16, False).startswith("decode")
    assert _lib.describe_plan(4, 128, 28672, 4096, 5, True) == "midbatch b4 g128 zp1 R4 mb1"
    # five to eight rows on layers with at most 512 row blocks: the gemv kernel's instantiation for eight
    # batch rows (one scale per tile or row; two row blocks per workgroup from 320 row blocks on)
    assert _lib.describe_plan(8, 128, 4096, 4096, 5, True) == "gemv b8 g128 zp1 T4 R1 W8 pad0"
    assert _lib.describe_plan(4, 128, 4096, 14336, 8, True) == "gemv b4 g128 zp1 T4 R1 W16 pad0"
    assert _lib.describe_plan(4, -1, 6144, 4096, 6, False) == "gemv b4 g-1 zp0 T4 R2 W8 pad0"
    assert _lib.describe_plan(4, 128, 8192, 28672, 8, True) == "gemv b4 g128 zp1 T4 R2 W15 pad0"  # (LDS: fifteen waves)
    assert _lib.describe_plan(6, 128, 8192, 8192, 8, True) == "midbatch b6 g128 zp1 R2 mb1"
    assert _lib.describe_plan(6, 128, 6144, 4096, 8, True) == "gemv b6 g128 zp1 T4 R2 W8 pad0"
    assert _lib.describe_plan(4, 128, 10240, 8192, 8, True).startswith("midbatch")
    assert _lib.describe_plan(4, 128, 4096, 4096, 9, True) == "midbatch b4 g128 zp1 R1 mb1"
    assert _lib.describe_plan(8, 32, 4096, 4096, 5, True) == "midbatch b8 g32 zp1 R1 mb1"
    assert _lib.describe_plan(4, 128, 8192, 8192, 2048).startswith("prefill")
    with pytest.raises(RuntimeError):
        _lib.describe_plan(4, 128, 4096, 4096, 1, True, 1 | (107 << 8))   # no such gemv entry
    with pytest.raises(RuntimeError):
        _lib.describe_plan(4, 128, 4096, 4096, 1, True, 1 | (100 << 8) | (17 << 18))  # more than 16 waves
    with pytest.raises(RuntimeError):
        _lib.describe_plan(4, 128, 4096, 4096, 1, True, 1 | (100 << 8) | (41 << 23))  # more LDS than a CU has
    assert _lib.describe_plan(8, 128, 28672, 4096, 16, True).startswith("decode")
    assert _lib.describe_plan(4, 128, 28672, 4096, 16, True) == "midbatch b4 g128 zp1 R4 mb1"
    # small layers: the mid-batch kernel (K split inside the workgroup) from a few rows on
    assert _lib.describe_plan(4, 128, 4096, 4096, 16, True).startswith("midbatch")
    assert _lib.describe_plan(4, 32, 4096, 14336, 5, True).startswith("midbatch")
    assert _lib.describe_plan(3, 32, 16, 1024, 17).startswith("midbatch")
    assert _lib.describe_plan(4, 128, 4096, 4096, 128, True) == "midbatch b4 g128 zp1 R4 mb2"
    assert _lib.describe_plan(8, 128, 4096, 4096, 128, True) == "midbatch b8 g128 zp1 R2 mb4"
    assert _lib.describe_plan(4, 128, 28672, 4096, 128, True).startswith("prefill")
    assert _lib.describe_plan(4, 128, 4096, 4096, 16, True, 1 | (1 << 8)).startswith("decode")


def test_planner_takes_the_tail_split_for_a_fraction_of_a_round():
    # 640 tiles of 128 x 256 are one round of 512 resident workgroups and a quarter: the rows of
    # the quarter go to narrower tiles; whole rounds keep the plain tile
    assert _lib.describe_plan(4, 128, 10240, 8192, 2048, True).endswith("cfg12")
    assert _lib.describe_plan(4, 128, 8192, 8192, 2048, True).endswith("cfg0")
    assert _lib.describe_plan(4, 128, 57344, 8192, 2048, True).endswith("cfg0")
    # behind one whole round the cheapest tail by workgroup counts: a round and five eighths (320 wide
    # tiles left, or 640 of 128 rows, or 432 of 192 rows) ends on 128 x 192 tiles
    assert _lib.describe_plan(4, 128, 13312, 8192, 2048, True).endswith("cfg15")
    # 28672 x 4096 behind its one round: 216 tiles of 192 rows sit alone on their CUs (M = 768), 100 of
    # 128 rows run K split (M = 640), 364 of 192 rows beat 273 wide and 546 narrow ones (M = 896)
    assert _lib.describe_plan(4, 128, 28672, 4096, 768, True).endswith("cfg15")
    assert _lib.describe_plan(4, 128, 28672, 4096, 640, True).endswith("cfg12")
    assert _lib.describe_plan(4, 128, 28672, 4096, 896, True).endswith("cfg15")


def test_planner_mixes_the_widest_tile_with_192_rows_where_one_round_of_it_leaves_slots_empty():
    # 448 tiles of 128 x 256 on 512 slots, 600 of 128 x 192: 256 of the first and 256 of the second
    assert _lib.describe_plan(4, 128, 28672, 4096, 512, True).endswith("cfg17")
    assert _lib.describe_plan(4, 128, 14336, 8192, 1024, True).endswith("cfg17")
    assert _lib.describe_plan(4, 128, 28672, 4096, 512, True, 1 | (90 << 8)).endswith("cfg17")
    # formats that do not take the 128 x 256 tile keep their own choice
    assert not _lib.describe_plan(6, 128, 28672, 4096, 512, True).endswith("cfg17")
    assert not _lib.describe_plan(4, 32, 28672, 4096, 512, True).endswith("cfg17")
    # the mixes need their wide tiles to number at most the CUs: 324 of 192 rows here, so 192 rows alone
    assert _lib.describe_plan(4, 128, 28672, 4096, 384, True).endswith("cfg9")
    # a few more 128 x 256 tiles than CUs (280) are a large batch too: one round of two widths
    assert _lib.describe_plan(4, 128, 14336, 8192, 640, True).endswith("cfg14")
    assert _lib.describe_plan(4, 128, 10240, 8192, 896, True).endswith("cfg14")


def test_planner_gives_three_quarters_of_a_round_to_192_row_tiles():
    # behind the whole rounds, rows that would be three quarters of a round of the wide tile (and more
    # than a round of 128 x 128 tiles) are one round of 128 x 192 tiles
    assert _lib.describe_plan(4, 128, 14336, 8192, 2048, True).endswith("cfg15")
    assert _lib.describe_plan(4, 128, 57344, 8192, 512, True).endswith("cfg15")
    assert _lib.describe_plan(4, 128, 28672, 4096, 1024, True).endswith("cfg15")
    for bits in (2, 3, 8):
        assert _lib.describe_plan(bits, 128, 14336, 8192, 2048, True).endswith("cfg15")
    assert _lib.describe_plan(4, 128, 14336, 8192, 2048, True, 3).endswith("cfg15")   # bf16 storage at 4 bits
    assert not _lib.describe_plan(6, 128, 14336, 8192, 2048, True).endswith("cfg15")  # formats with a tile rule of their own
    assert not _lib.describe_plan(4, 32, 14336, 8192, 2048, True).endswith("cfg15")
    # far from a whole round of them, or nothing behind the whole rounds: the plain tile
    assert _lib.describe_plan(4, 128, 57344, 8192, 768, True).endswith("cfg0")
    assert _lib.describe_plan(4, 128, 57344, 8192, 2048, True).endswith("cfg0")


def test_planner_keeps_small_batches_on_very_wide_layers_off_the_padded_tiles():
    # a vocabulary-sized layer fills the 128 x 256 tiles' slots at any batch size; up to 64 batch rows
    # those tiles would be mostly padding
    assert _lib.describe_plan(4, 128, 128256, 4096, 32, True).endswith("cfg4")
    assert _lib.describe_plan(4, 128, 128256, 4096, 17, True).endswith("cfg4")
    assert _lib.describe_plan(4, 128, 128256, 4096, 128, True).endswith("cfg0")
    assert _lib.describe_plan(4, 128, 128256, 4096, 2048, True).endswith("cfg0")


def test_planner_takes_192_row_tiles_where_they_fill_one_round_better():
    # 6144 rows at M = 2048: 384 tiles of 128 x 256 leave half the CUs with one workgroup, 512 tiles
    # of 128 x 192 fill every slot; past 512 of them the wide tile is back
    for bits in (2, 3, 4, 8):
        assert _lib.describe_plan(bits, 128, 6144, 4096, 2048, True).endswith("cfg9")
    assert _lib.describe_plan(4, 32, 6144, 4096, 2048, False).endswith("cfg9")
    assert _lib.describe_plan(4, 128, 6144, 4096, 2560, True).endswith("cfg0")
    assert _lib.describe_plan(4, 128, 7168, 4096, 2048, True).endswith("cfg17")  # 448 wide tiles: mixed with 192 rows


def test_planner_mixes_two_tile_widths_where_neither_fills_the_one_round():
    # 5120 rows at M = 2048: 32 slots per column of activation tiles; 27 tiles of 192 rows leave five
    # empty, 40 of 128 rows need a second round: 16 of 192 and 16 of 128 take every slot once
    assert _lib.describe_plan(4, -1, 5120, 4096, 2048, True).endswith("cfg14")
    for bits in (2, 3, 4, 8):
        assert _lib.describe_plan(bits, 128, 10240, 8192, 1024, True).endswith("cfg14")
    assert _lib.describe_plan(4, 128, 10240, 8192, 1024, False).endswith("cfg14")
    assert _lib.describe_plan(4, 128, 10240, 8192, 1024, True, 3).endswith("cfg14")  # bf16 storage at 4 bits
    # formats that do not take the 128 x 192 tile in that regime keep their own choice
    assert not _lib.describe_plan(6, 128, 10240, 8192, 1024, True).endswith("cfg14")
    assert not _lib.describe_plan(4, 32, 10240, 8192, 1024, True).endswith("cfg14")
    # exactly one round of 128 x 192 tiles, or of 128 x 128 tiles: no mix
    assert _lib.describe_plan(4, 128, 6144, 4096, 2048, True).endswith("cfg9")
    assert not _lib.describe_plan(4, 128, 8192, 8192, 1024, True).endswith("cfg14")


def test_planner_splits_k_in_the_workgroup_where_ring_tiles_would_sit_one_per_cu():
    # 128 x 128 tiles that number at most the CUs: eight waves per workgroup, K in two halves
    assert _lib.describe_plan(4, 128, 8192, 8192, 512, True).endswith("cfg10")
    assert _lib.describe_plan(4, 128, 28672, 4096, 128, True).endswith("cfg10")
    assert _lib.describe_plan(4, 32, 8192, 8192, 512, True).endswith("cfg10")      # every format fits it
    assert _lib.describe_plan(4, 128, 8192, 8192, 512, True, 3).endswith("cfg10")  # bf16 storage too
    # more of those than CUs but at most as many 128 x 256 tiles: the wide tile, split
    assert _lib.describe_plan(4, 128, 8192, 8192, 1024, True).endswith("cfg11")
    assert _lib.describe_plan(4, 128, 10240, 8192, 768, True).endswith("cfg11")
    # 128 x 192 tiles, split the same way, where they put more of the CUs to work in the one round
    assert _lib.describe_plan(4, 128, 10240, 8192, 512, True).endswith("cfg13")
    assert _lib.describe_plan(8, 128, 8192, 8192, 1024, True).endswith("cfg11")
    assert _lib.describe_plan(6, 128, 8192, 8192, 1024, True).endswith("cfg3")     # 6 bits: registers
    assert _lib.describe_plan(3, 128, 8192, 8192, 1024, True, 3).endswith("cfg3")  # 3 bits on bf16 storage likewise
    assert _lib.describe_plan(4, 128, 8192, 8192, 1024, True, 3).endswith("cfg11")
    assert _lib.describe_plan(8, 128, 8192, 8192, 1024, True, 3).endswith("cfg11")
    # short K walks as well, down to where the small staged tile fits one round
    assert _lib.describe_plan(4, 128, 4096, 2048, 1024, True).endswith("cfg10")
    assert _lib.describe_plan(4, 128, 4096, 1024, 1024, True).endswith("cfg10")
    assert _lib.describe_plan(4, 128, 4096, 1024, 512, True).endswith("cfg4")


def test_planner_takes_64_row_split_tiles_where_128_row_ones_leave_half_of_the_cus_idle():
    # 64 x 128 tiles, K in two halves inside the workgroup, while they number at most the CUs
    assert _lib.describe_plan(4, 128, 4096, 4096, 512, True).endswith("cfg16")
    assert _lib.describe_plan(4, 128, 6144, 4096, 256, True).endswith("cfg16")
    assert _lib.describe_plan(4, 128, 4096, 14336, 512, True).endswith("cfg16")
    assert _lib.describe_plan(4, 128, 28672, 4096, 64, True).endswith("cfg16")
    assert _lib.describe_plan(4, 32, 4096, 4096, 512, True).endswith("cfg16")      # every format
    assert _lib.describe_plan(4, -1, 4096, 4096, 512, False).endswith("cfg16")
    assert _lib.describe_plan(4, 128, 4096, 4096, 512, True, 3).endswith("cfg16")  # bf16 storage
    assert _lib.describe_plan(8, 128, 6144, 4096, 192, True).endswith("cfg16")
    # more of them than CUs: the 128-row tile
    assert _lib.describe_plan(4, 128, 6144, 4096, 384, True).endswith("cfg10")
    assert _lib.describe_plan(4, 128, 4096, 14336, 768, True).endswith("cfg10")
    assert _lib.describe_plan(4, 128, 28672, 4096, 128, True).endswith("cfg10")
    # smaller batches stay with the mid-batch kernel while its workgroups fit their rounds
    assert _lib.describe_plan(4, 128, 4096, 4096, 192, True).startswith("midbatch")
    assert _lib.describe_plan(8, 128, 6144, 4096, 96, True).startswith("midbatch")
    # the forced variant: 89
    assert _lib.describe_plan(4, 128, 8192, 8192, 2048, True, 1 | (89 << 8)).endswith("cfg16")
    with pytest.raises(_lib.MatGPTQError):
        _lib.describe_plan(4, 128, 8192, 8192, 2048, True, 1 | (92 << 8))


def test_planner_gives_eight_row_blocks_to_32_batch_rows_on_layers_with_many_rows():
    # the mid-batch kernel with eight row blocks and 32 batch rows per workgroup where that leaves 200 workgroups
    assert _lib.describe_plan(4, 128, 28672, 4096, 32, True) == "midbatch b4 g128 zp1 R8 mb2"
    assert _lib.describe_plan(2, 128, 28672, 4096, 24, True) == "midbatch b2 g128 zp1 R8 mb2"
    assert _lib.describe_plan(4, 128, 28672, 4096, 32, True, 3) == "midbatch b4 g128 zp1 R8 mb2"  # bf16 storage
    assert _lib.describe_plan(4, 128, 10240, 8192, 32, True) == "midbatch b4 g128 zp1 R4 mb2"     # 80 workgroups only
    assert _lib.describe_plan(6, 128, 28672, 4096, 32, True) == "midbatch b6 g128 zp1 R4 mb2"     # registers
    assert _lib.describe_plan(4, 128, 28672, 4096, 16, True) == "midbatch b4 g128 zp1 R4 mb1"


def test_planner_keeps_group_32_with_zero_points_off_the_largest_ring_tile():
    # four scales and four zeros per tile and row block in two register sets spill there
    assert _lib.describe_plan(4, 32, 8192, 8192, 2048, True).endswith("cfg3")
    assert _lib.describe_plan(8, 32, 8192, 8192, 2048, True).endswith("cfg3")
    assert _lib.describe_plan(4, 32, 57344, 8192, 2048, True).endswith("cfg9")
    assert _lib.describe_plan(6, 32, 57344, 8192, 2048, True).endswith("cfg3")
    assert _lib.describe_plan(4, 32, 8192, 8192, 2048, False).endswith("cfg0")   # scales alone fit
    assert _lib.describe_plan(4, -1, 8192, 8192, 2048, True).endswith("cfg0")


def test_planner_gives_bf16_storage_the_wide_ring_tile_where_its_registers_hold():
    # bf16 weights are formed in fp32 (four vector instructions per pair instead of three).  2- and 4-bit
    # codes, and 8-bit codes with one scale per row, follow the rules of fp16 storage; the others spill in
    # the 128 x 256 tile: 128 x 192 where its rounds pay (not at 6 bits: registers), else 128 x 128, and
    # 8-bit codes the 128 x 256 tile split over eight waves up to two rounds of them.  Every tile can be forced.
    for bits in (2, 4):
        for zp in (True, False):
            assert _lib.describe_plan(bits, 128, 10240, 8192, 2048, zp, 3) == _lib.describe_plan(bits, 128, 10240, 8192, 2048, zp, 1)
            assert _lib.describe_plan(bits, 128, 57344, 8192, 2048, zp, 3).endswith("cfg0")
            assert _lib.describe_plan(bits, -1, 8192, 28672, 2048, zp, 3).endswith("cfg0")
    assert _lib.describe_plan(4, 128, 10240, 8192, 1024, True, 3).endswith("cfg14")  # (both widths in one launch)
    assert _lib.describe_plan(8, -1, 8192, 8192, 2048, True, 3).endswith("cfg0")
    assert _lib.describe_plan(4, 32, 8192, 8192, 2048, False, 3).endswith("cfg3")
    assert _lib.describe_plan(3, 128, 8192, 8192, 2048, True, 3).endswith("cfg3")
    assert _lib.describe_plan(3, 128, 10240, 8192, 2048, True, 3).endswith("cfg9")
    assert _lib.describe_plan(8, 128, 57344, 8192, 2048, True, 3).endswith("cfg9")
    assert _lib.describe_plan(8, 128, 8192, 8192, 2048, True, 3).endswith("cfg11")
    assert _lib.describe_plan(8, 128, 6144, 4096, 2048, True, 3).endswith("cfg9")
    assert _lib.describe_plan(6, 128, 57344, 8192, 2048, True, 3).endswith("cfg3")
    assert _lib.describe_plan(4, 128, 10240, 8192, 2048, True, 3 | (72 << 8)).endswith("cfg8")


def test_planner_six_and_eight_bit_codes_on_the_ring_tiles():
    # 6- and 8-bit codes keep one register set on the 128 x 256 tile, refilled octet by octet; 6-bit codes
    # take it where its tiles fill whole rounds (fp16 storage, one scale per tile or row)
    assert _lib.describe_plan(6, 128, 8192, 8192, 2048, True).endswith("cfg0")
    assert _lib.describe_plan(6, 128, 28672 // 4, 8192, 2048, False).endswith("cfg0")
    assert _lib.describe_plan(6, 32, 8192, 8192, 2048, False).endswith("cfg3")
    assert _lib.describe_plan(6, 128, 8192, 8192, 2048, True, 3).endswith("cfg3")  # bf16 storage: registers
    assert _lib.describe_plan(6, 128, 10240, 8192, 2048, False).endswith("cfg9")  # 54 tiles of 192 rows: two rounds
    # many rounds: the 128 x 192 tile, which still fits the registers
    assert _lib.describe_plan(6, 128, 57344, 8192, 2048, True).endswith("cfg9")
    assert _lib.describe_plan(8, 128, 57344, 8192, 2048, True).endswith("cfg0")
    assert _lib.describe_plan(8, 128, 57344, 8192, 2048, False).endswith("cfg0")
    assert _lib.describe_plan(8, 128, 8192, 8192, 2048, True).endswith("cfg0")
    assert _lib.describe_plan(8, 128, 10240, 8192, 2048, True).endswith("cfg12")
    assert _lib.describe_plan(8, 128, 8192, 8192, 2048, False).endswith("cfg0")
    assert _lib.describe_plan(3, 128, 8192, 8192, 2048, True).endswith("cfg0")


def test_header_is_plain_c(tmp_path):
    # the boundary is a C ABI: the header has to compile as C99 with nothing but the standard headers
    import shutil
    import subprocess
    cc = shutil.which("gcc") or shutil.which("cc")
    if cc is None:
        pytest.skip("no C compiler")
    src = tmp_path / "t.c"
    src.write_text('#include "matgptq_abi.h"\nint main(void) { return matgptq_abi_version() == 0; }\n')
    subprocess.run([cc, "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(ROOT, "include"),
                    "-c", str(src), "-o", str(tmp_path / "t.o")], check=True)


def test_planner_answers_every_valid_shape_within_its_kernels_domains():
    # seeded random problems: a plan for each, the gemv kernel only up to eight batch rows (five to
    # eight: one scale per tile or row, at most 512 row blocks, waves within the LDS of a CU), the
    # mid-batch kernel from five rows on, the large-batch tiles from seventeen
    import random
    import re
    rnd = random.Random(7)
    seen = set()
    for _ in range(6000):
        b = rnd.choice((2, 3, 4, 6, 8))
        g = rnd.choice((128, 32, -1))
        n = 16 * rnd.choice((1, 2, 5, 16, 64, 255, 256, 319, 320, 384, 512, 513, 640, 1024, 1792, 3584, 8016))
        k = 128 * rnd.choice((1, 2, 3, 4, 7, 8, 16, 31, 32, 64, 112, 224)) + (64 if g != 128 and rnd.random() < 0.1 else 0)
        m = rnd.choice((1, 2, 3, 4, 5, 6, 7, 8, 9, 15, 16, 17, 31, 32, 33, 64, 100, 128, 129, 256, 384, 512, 1000, 1024, 2048, 4096))
        flags = 1 | (2 if rnd.random() < 0.3 else 0)
        if k % 128 == 64 and k < 192:
            continue
        plan = _lib.describe_plan(b, g, n, k, m, rnd.random() < 0.5, flags)
        kind = plan.split()[0]
        seen.add(kind)
        if kind == "gemv":
            assert m <= 8, plan
            w, r, t = (int(re.search(rf" {c}(\d+)", plan).group(1)) for c in "WRT")
            assert 1 <= w <= 16, plan
            if m > 4:
                assert g != 32 and n // 16 <= 512, plan
                assert w * (8 * (t * 256 + 16) + 256 + 64 * t + r * 1024) <= 160 * 1024, plan
        elif kind == "midbatch":
            assert m > 4, plan
        elif kind == "prefill":
            assert m > 16, plan
        else:
            assert kind.startswith("decode") and m <= 16, plan
    assert {"gemv", "midbatch", "prefill"} <= seen
