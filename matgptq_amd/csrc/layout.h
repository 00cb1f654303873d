// Packed weight layout of the gfx950 kernels, shared by host packers and device code.
//
// The [N, K] matrix of b-bit codes is cut into TILES of 16 rows x 128 columns.
// Tiles are stored row-block major: tile (rb, kb) starts at word
// (rb * K/128 + kb) * 64*b.  One tile is exactly what one 64-lane wavefront
// consumes per step:
//
//   lane l  ->  row  r = l % 16,   k-quarter  q = l / 16
//   the lane owns 32 codes, grouped in four OCTETS j = 0..3 of eight codes e = 0..7:
//       k = kb*128 + j*32 + q*8 + e
//
// so that octet j of all 64 lanes is a 16 x 32 operand of one
// v_mfma_f32_16x16x32_f16 (row = l % 16, eight consecutive k per lane), and
// octet j covers the contiguous column range [kb*128 + j*32, +32).
//
// A tile is a sequence of SEGMENTS; a segment holds 1, 2 or 4 consecutive words
// per lane, lane-major, so every segment is read by one fully coalesced
// global_load_dword / dwordx2 / dwordx4 of the wavefront:
//
//   b = 2 : [ 2 words/lane ]                      word d = octets 2d, 2d+1 (2-bit fields)
//   b = 3 : [ 2 words/lane | 1 word/lane ]        low two bits as for b=2-style planes, bit 2
//   b = 4 : [ 4 words/lane ]                      word j = octet j (nibbles)
//   b = 6 : [ 4 words/lane | 2 words/lane ]       high four bits as b=4, low two bits
//   b = 8 : [ 4 words/lane | 4 words/lane ]       words 2j, 2j+1 = octet j (bytes)
//
// Total size is b*N*K/32 words, the size the reference's op contract exposes
// (inference_lib/matgptq_cuda/csrc/bindings.cpp:68,160); the byte order inside
// is private, as it is in the reference.
//
// K = 128 t + 64 (group sizes 32 and -1 only; the reference packs any K % 64 == 0,
// inference_lib/matgptq_cuda/csrc/utils.cpp:174-184): the t tiles of every row block come first,
// as above with K/128 = t; the last 64 columns of all rows (the TAIL) follow them as plain
// bitstreams, 2 b words per row, code k of a row at bit k * b.  Still b*N*K/32 words.
//
// Inside a word the fields are permuted so that a mask, an OR with 0x6400 and
// at most one shift leave two codes as the low mantissa bits of a packed pair
// of fp16 numbers 1024 + c * 2^p.  `decode_octet` below produces these "raw"
// pairs; element 2i of the octet is the low half of pair i, element 2i+1 the
// high half.  `kRawShift<b>(i)` gives p for pair i.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define MATGPTQ_HD __host__ __device__ __forceinline__
#else
#define MATGPTQ_HD inline
#endif

namespace matgptq {

constexpr int kTileRows = 16;
constexpr int kTileCols = 128;
constexpr int kLanes = 64;
constexpr uint32_t kMagic = 0x64006400u;  // two fp16 1024.0

constexpr bool valid_bits(int b) { return b == 2 || b == 3 || b == 4 || b == 6 || b == 8; }
constexpr bool valid_group(int g) { return g == -1 || g == 32 || g == 128; }
constexpr int tile_words(int b) { return 64 * b; }

// The tail of K = 128 t + 64.
constexpr int kTailCols = 64;
constexpr int tail_row_words(int b) { return 2 * b; }
// K is a multiple of 128, or such a multiple (at least one tile) plus 64
constexpr bool valid_k(int64_t K) { return K > 0 && (K % 128 == 0 || (K % 128 == 64 && K >= 192)); }
// code k (0..63) of a tail row stored at `row` (2 b words)
MATGPTQ_HD uint32_t tail_code(const uint32_t* row, int b, int k) {
  const int bit = k * b, w = bit >> 5, sh = bit & 31;
  uint32_t v = row[w] >> sh;
  if (sh + b > 32) v |= row[w + 1] << (32 - sh);
  return v & ((1u << b) - 1u);
}
// 64 codes -> the 2 b words of a tail row
MATGPTQ_HD void tail_encode_row(const uint8_t* codes, int b, uint32_t* row) {
  for (int i = 0; i < 2 * b; i++) row[i] = 0u;
  for (int k = 0; k < kTailCols; k++) {
    const uint32_t c = (uint32_t)codes[k] & ((1u << b) - 1u);
    const int bit = k * b, w = bit >> 5, sh = bit & 31;
    row[w] |= c << sh;
    if (sh + b > 32) row[w + 1] |= c >> (32 - sh);
  }
}

// Number of words of the first segment per lane; the second segment (if any)
// holds the remaining words.
constexpr int seg0_words(int b) { return b == 2 ? 2 : b == 3 ? 2 : 4; }
constexpr int seg1_words(int b) { return b == 3 ? 1 : b == 6 ? 2 : b == 8 ? 4 : 0; }

// Word offset, inside a tile, of word `w` (0 <= w < b) of lane `lane`.
MATGPTQ_HD int word_offset(int b, int lane, int w) {
  const int s0 = seg0_words(b);
  if (w < s0) return lane * s0 + w;
  const int s1 = seg1_words(b);
  return kLanes * s0 + lane * s1 + (w - s0);
}

// ----- nibble word (eight 4-bit fields) ---------------------------------
// Octet element e sits in nibble kNibbleOf[e], so that
//   x        & 0x000F000F -> (e0, e1)      x        & 0x00F000F0 -> (e2, e3) << 4
//   (x >> 8) & 0x000F000F -> (e4, e5)      (x >> 8) & 0x00F000F0 -> (e6, e7) << 4
MATGPTQ_HD int nibble_of(int e) {
  // e: 0 1 2 3 4 5 6 7  ->  0 4 1 5 2 6 3 7
  return (e >> 1) + ((e & 1) << 2);
}

// Raw pairs of a nibble word: r[i] = 1024 + c << p(i), p = {0, 4, 0, 4}.
MATGPTQ_HD void raw_from_nibbles(uint32_t x, uint32_t (&r)[4]) {
  const uint32_t x8 = x >> 8;
  r[0] = (x & 0x000F000Fu) | kMagic;
  r[1] = (x & 0x00F000F0u) | kMagic;
  r[2] = (x8 & 0x000F000Fu) | kMagic;
  r[3] = (x8 & 0x00F000F0u) | kMagic;
}

template <int BITS>
struct Codec;

// ----- b = 4 --------------------------------------------------------------
template <>
struct Codec<4> {
  static constexpr int kCentre = 8;
  static constexpr int raw_shift(int /*j*/, int i) { return (i & 1) ? 4 : 0; }
  MATGPTQ_HD static void decode_octet(const uint32_t (&w)[4], int j, uint32_t (&r)[4]) {
    raw_from_nibbles(w[j], r);
  }
  // codes: the lane's 32 codes, index j*8 + e
  MATGPTQ_HD static void encode_lane(const uint8_t (&codes)[32], uint32_t (&w)[4]) {
    for (int j = 0; j < 4; j++) {
      uint32_t x = 0;
      for (int e = 0; e < 8; e++) x |= (uint32_t)(codes[j * 8 + e] & 0xF) << (4 * nibble_of(e));
      w[j] = x;
    }
  }
};

// ----- b = 2 --------------------------------------------------------------
// Word d holds octets 2d and 2d+1 as sixteen 2-bit fields.  In each 16-bit half
// field f (bits 2f, 2f+1) belongs to pair f: pairs 0..3 are octet 2d, pairs
// 4..7 octet 2d+1; the low half holds the even element, the high half the odd.
// Fields 0..2 are read in place, 3..5 after a shift by 6, 6..7 after a shift by
// 12, so that no field sits higher than bit 4 of the mantissa (p <= 4).
template <>
struct Codec<2> {
  static constexpr int kCentre = 2;
  static constexpr int raw_shift(int j, int i) {
    const int f = (j & 1) * 4 + i;  // field index in the half word
    return 2 * (f % 3);
  }
  MATGPTQ_HD static void decode_octet(const uint32_t (&w)[2], int j, uint32_t (&r)[4]) {
    const uint32_t x = w[j >> 1];
    const uint32_t x6 = x >> 6;
    if ((j & 1) == 0) {
      r[0] = (x & 0x00030003u) | kMagic;
      r[1] = (x & 0x000C000Cu) | kMagic;
      r[2] = (x & 0x00300030u) | kMagic;
      r[3] = (x6 & 0x00030003u) | kMagic;
    } else {
      const uint32_t x12 = x >> 12;
      r[0] = (x6 & 0x000C000Cu) | kMagic;
      r[1] = (x6 & 0x00300030u) | kMagic;
      r[2] = (x12 & 0x00030003u) | kMagic;
      r[3] = (x12 & 0x000C000Cu) | kMagic;
    }
  }
  MATGPTQ_HD static void encode_lane(const uint8_t (&codes)[32], uint32_t (&w)[2]) {
    for (int d = 0; d < 2; d++) {
      uint32_t x = 0;
      for (int f = 0; f < 8; f++) {
        const int j = 2 * d + (f >> 2), i = f & 3;
        x |= (uint32_t)(codes[j * 8 + 2 * i] & 3) << (2 * f);
        x |= (uint32_t)(codes[j * 8 + 2 * i + 1] & 3) << (2 * f + 16);
      }
      w[d] = x;
    }
  }
};

// ----- b = 8 --------------------------------------------------------------
// Words 2j, 2j+1 hold octet j.  In word 2j+d: byte0 = e(4d), byte2 = e(4d+1),
// byte1 = e(4d+2), byte3 = e(4d+3), so that
//   x & 0x00FF00FF -> pair 2d,   (x >> 8) & 0x00FF00FF -> pair 2d+1.
template <>
struct Codec<8> {
  static constexpr int kCentre = 128;
  static constexpr int raw_shift(int, int) { return 0; }
  MATGPTQ_HD static void decode_octet(const uint32_t (&w)[8], int j, uint32_t (&r)[4]) {
    const uint32_t a = w[2 * j], b = w[2 * j + 1];
    r[0] = (a & 0x00FF00FFu) | kMagic;
    r[1] = ((a >> 8) & 0x00FF00FFu) | kMagic;
    r[2] = (b & 0x00FF00FFu) | kMagic;
    r[3] = ((b >> 8) & 0x00FF00FFu) | kMagic;
  }
  MATGPTQ_HD static void encode_lane(const uint8_t (&codes)[32], uint32_t (&w)[8]) {
    for (int j = 0; j < 4; j++)
      for (int d = 0; d < 2; d++) {
        const uint8_t* c = &codes[j * 8 + 4 * d];
        w[2 * j + d] = (uint32_t)c[0] | ((uint32_t)c[2] << 8) | ((uint32_t)c[1] << 16) |
                       ((uint32_t)c[3] << 24);
      }
  }
};

// ----- b = 3 --------------------------------------------------------------
// Words 0,1: the low two bits of every code; word d serves octets 2d, 2d+1 and
// nibble n of it is  [octet 2d low2 | octet 2d+1 low2 << 2]  for the element that
// lives in nibble n of a b=4 word.  Word 2: bit 2 of every code; nibble n holds the
// bits of octets 0..3 at bit positions 0..3.  An octet is rebuilt as a nibble word
// and then decoded like b = 4.
template <>
struct Codec<3> {
  static constexpr int kCentre = 4;
  static constexpr int raw_shift(int, int i) { return (i & 1) ? 4 : 0; }
  MATGPTQ_HD static uint32_t nibble_word(const uint32_t (&w)[3], int j) {
    const uint32_t lo = (w[j >> 1] >> (2 * (j & 1))) & 0x33333333u;
    const uint32_t c = w[2];
    const uint32_t hi = (j == 0 ? (c << 2) : j == 1 ? (c << 1) : j == 2 ? c : (c >> 1)) & 0x44444444u;
    return lo | hi;
  }
  MATGPTQ_HD static void decode_octet(const uint32_t (&w)[3], int j, uint32_t (&r)[4]) {
    raw_from_nibbles(nibble_word(w, j), r);
  }
  MATGPTQ_HD static void encode_lane(const uint8_t (&codes)[32], uint32_t (&w)[3]) {
    w[0] = w[1] = w[2] = 0;
    for (int j = 0; j < 4; j++)
      for (int e = 0; e < 8; e++) {
        const uint32_t c = codes[j * 8 + e] & 7;
        const int n = nibble_of(e);
        w[j >> 1] |= (c & 3) << (4 * n + 2 * (j & 1));
        w[2] |= (c >> 2) << (4 * n + j);
      }
  }
};

// ----- b = 6 --------------------------------------------------------------
// Words 0..3: the high four bits of every code, laid out as a b=4 tile.
// Words 4,5: the low two bits; word 4+d serves octets 2d (u = 0) and 2d+1 (u = 1).
// With s = 8u the low bits of pair 0 sit at bits s+0..1, of pair 2 at s+2..3, of
// pair 1 at s+4..5 and of pair 3 at s+6..7 (odd elements 16 bits higher), so that
// after  (hi_field << 2) | lo_field  pairs 0, 2 read 1024 + c and pairs 1, 3 read
// 1024 + 16c.
template <>
struct Codec<6> {
  static constexpr int kCentre = 32;
  static constexpr int raw_shift(int, int i) { return (i & 1) ? 4 : 0; }
  MATGPTQ_HD static void decode_octet(const uint32_t (&w)[6], int j, uint32_t (&r)[4]) {
    const uint32_t h = w[j], h8 = h >> 8;
    const uint32_t l = w[4 + (j >> 1)] >> (8 * (j & 1));
    const uint32_t l2 = l >> 2;
    r[0] = ((h & 0x000F000Fu) << 2) | (l & 0x00030003u) | kMagic;
    r[1] = ((h & 0x00F000F0u) << 2) | (l & 0x00300030u) | kMagic;
    r[2] = ((h8 & 0x000F000Fu) << 2) | (l2 & 0x00030003u) | kMagic;
    r[3] = ((h8 & 0x00F000F0u) << 2) | (l2 & 0x00300030u) | kMagic;
  }
  MATGPTQ_HD static void encode_lane(const uint8_t (&codes)[32], uint32_t (&w)[6]) {
    for (int i = 0; i < 6; i++) w[i] = 0;
    // bit offset of pair i's low field inside an 8-bit group: pairs 0,2,1,3 -> 0,2,4,6
    const int lo_off[4] = {0, 4, 2, 6};
    for (int j = 0; j < 4; j++)
      for (int e = 0; e < 8; e++) {
        const uint32_t c = codes[j * 8 + e] & 63;
        w[j] |= (c >> 2) << (4 * nibble_of(e));
        const int pair = e >> 1, odd = e & 1;
        w[4 + (j >> 1)] |= (c & 3) << (8 * (j & 1) + lo_off[pair] + 16 * odd);
      }
  }
};

// Code of element e (0..7) of an octet from its raw pairs (host-side inverse).
template <int BITS>
MATGPTQ_HD uint8_t code_from_raw(const uint32_t (&r)[4], int j, int e) {
  const int i = e >> 1;
  const uint32_t half = (e & 1) ? (r[i] >> 16) : (r[i] & 0xFFFFu);
  return (uint8_t)((half & 0x3FFu) >> Codec<BITS>::raw_shift(j, i));
}

// Rounded MSB slice of an 8-bit master code (the reference's matryoshka_slice,
// src/quant_utils_matgpqt.py:9-17, with master_bitwidth = 8).
MATGPTQ_HD uint8_t slice_code(uint8_t q, int bits) {
  if (bits >= 8) return q;
  const int drop = 8 - bits;
  const int v = (q >> drop) + ((q >> (drop - 1)) & 1);
  const int top = (1 << bits) - 1;
  return (uint8_t)(v > top ? top : v);
}

}  // namespace matgptq
