// Master-resident layout: the 8-bit master codes stored as bit planes, most significant
// first, so that a kernel working at bitwidth b reads only the top b bits of every code plus
// the one bit below them and forms the reference's rounded slice
// (src/quant_utils_matgpqt.py:9-17:  min((q >> (8-b)) + ((q >> (7-b)) & 1), 2^b - 1))
// in registers.  One buffer serves every bitwidth; no counterpart in the reference, which
// slices on the host once and deletes the master codes (inference_lib/vllm_matgptq.py:154-178).
//
// Tiles are the 16 x 128 tiles of layout.h in the same order; a tile is 512 words (2 KiB).
// A lane (row l % 16, k-quarter l / 16) owns the same 32 codes, octet j, element e, as there.
// Its eight words, in plane order:
//     0,1  bits 7..6   word d serves octets 2d (u = 0) and 2d+1 (u = 1):
//                      bits [4 nb + 2u, +2) = the field of element e,  nb = nibble_of(e)
//     2    bit 5       bit 4 nb + j = the bit of element e of octet j
//     3    bit 4       as word 2
//     4    bit 3       as word 2
//     5    bit 2       as word 2
//     6,7  bits 1..0   as words 0,1
// stored as four segments, lane-major inside each, so that a bitwidth reads a prefix of the
// tile with fully coalesced loads of 12, 4, 4 and 12 bytes per lane:
//     S0 = words 0,1,2    S1 = word 3    S2 = word 4    S3 = words 5,6,7
//     b = 2 reads S0 (3 bits per weight), 3: S0 S1 (4 bits), 4: S0 S1 S2 (5 bits), 6 and 8: all.
//
// The positions are chosen so that a shift and a mask put a plane's bits of one octet at the
// same position in every nibble (b <= 4) or every byte (b >= 6) of a register word:
//     nibble word of octet j : nibble nb holds the sliced code of the element with nibble_of(e) = nb
//     byte word h of octet j : byte i holds the sliced code of the element with nibble_of(e) = 2 i + h
// and the rounding add and the saturation are done on all fields of a word at once.
#pragma once
#include "layout.h"

namespace matgptq {

constexpr int kMasterTileWords = 512;

// full unrolling of the small loops below in device code: left rolled, the word a plane's bits go to
// is picked by a chain of compares and selects per code
#if defined(__clang__)
#define MATGPTQ_UNROLL _Pragma("unroll")
#else
#define MATGPTQ_UNROLL
#endif

// words a lane reads at bitwidth b
constexpr int master_words(int b) { return b == 2 ? 3 : b == 3 ? 4 : b == 4 ? 5 : 8; }

// word offset inside a tile of word w (0..7, plane order) of a lane
MATGPTQ_HD int master_word_offset(int lane, int w) {
  if (w < 3) return lane * 3 + w;
  if (w == 3) return 192 + lane;
  if (w == 4) return 256 + lane;
  return 320 + lane * 3 + (w - 5);
}

// the lane's 32 master codes (index j*8 + e) -> its eight words
MATGPTQ_HD void master_encode_lane(const uint8_t (&codes)[32], uint32_t (&w)[8]) {
  for (int i = 0; i < 8; i++) w[i] = 0;
  MATGPTQ_UNROLL
  for (int j = 0; j < 4; j++)
    MATGPTQ_UNROLL
    for (int e = 0; e < 8; e++) {
      const uint32_t c = codes[j * 8 + e];
      const int nb = nibble_of(e), d = j >> 1, u = j & 1;
      w[d] |= ((c >> 6) & 3u) << (4 * nb + 2 * u);
      w[2] |= ((c >> 5) & 1u) << (4 * nb + j);
      w[3] |= ((c >> 4) & 1u) << (4 * nb + j);
      w[4] |= ((c >> 3) & 1u) << (4 * nb + j);
      w[5] |= ((c >> 2) & 1u) << (4 * nb + j);
      w[6 + d] |= (c & 3u) << (4 * nb + 2 * u);
    }
}

// Sliced codes of octet J as a nibble word (BITS 2, 3, 4), from the words a lane reads at BITS.
template <int BITS, int J>
MATGPTQ_HD uint32_t master_nibble_word(const uint32_t* w) {
  static_assert(BITS == 2 || BITS == 3 || BITS == 4, "nibble form");
  constexpr uint32_t k1 = 0x11111111u;
  const uint32_t f76 = (w[J >> 1] >> (2 * (J & 1))) & 0x33333333u;
  const uint32_t b5 = (w[2] >> J) & k1;
  if constexpr (BITS == 2) {
    const uint32_t s = f76 + b5;          // 0 .. 4 per nibble
    return s - ((s >> 2) & k1);           // 4 -> 3
  } else if constexpr (BITS == 3) {
    const uint32_t b4 = (w[3] >> J) & k1;
    const uint32_t s = ((f76 << 1) | b5) + b4;  // 0 .. 8
    return s - ((s >> 3) & k1);                 // 8 -> 7
  } else {
    const uint32_t b4 = (w[3] >> J) & k1;
    const uint32_t b3 = (w[4] >> J) & k1;
    const uint32_t top = (f76 << 2) | (b5 << 1) | b4;
    // a nibble of 15 must not take the round bit: bit 3 of `full` is set exactly for those
    const uint32_t full = ((top & 0x77777777u) + k1) & top & 0x88888888u;
    return top + (b3 & ~(full >> 3));
  }
}

// Sliced codes of octet J, elements with nibble index 2 i + H, as byte word (BITS 6, 8).
template <int BITS, int J, int H>
MATGPTQ_HD uint32_t master_byte_word(const uint32_t* w) {
  static_assert(BITS == 6 || BITS == 8, "byte form");
  constexpr uint32_t k1 = 0x01010101u, k3 = 0x03030303u;
  constexpr int sh2 = 2 * (J & 1) + 4 * H, sh1 = J + 4 * H, d = J >> 1;
  const uint32_t f76 = (w[d] >> sh2) & k3;
  const uint32_t b5 = (w[2] >> sh1) & k1, b4 = (w[3] >> sh1) & k1;
  const uint32_t b3 = (w[4] >> sh1) & k1, b2 = (w[5] >> sh1) & k1;
  const uint32_t f10 = (w[6 + d] >> sh2) & k3;
  if constexpr (BITS == 8) {
    return (f76 << 6) | (b5 << 5) | (b4 << 4) | (b3 << 3) | (b2 << 2) | f10;
  } else {
    const uint32_t s = ((f76 << 4) | (b5 << 3) | (b4 << 2) | (b3 << 1) | b2) + ((f10 >> 1) & k1);  // 0 .. 64
    return s - ((s >> 6) & k1);                                                                     // 64 -> 63
  }
}

// The sliced code of element e of octet J (host checks, unpack kernels).
template <int BITS, int J>
MATGPTQ_HD uint8_t master_code(const uint32_t* w, int e) {
  const int nb = nibble_of(e);
  if constexpr (BITS <= 4) {
    return (uint8_t)((master_nibble_word<BITS, J>(w) >> (4 * nb)) & 0xFu);
  } else {
    const uint32_t word = (nb & 1) ? master_byte_word<BITS, J, 1>(w) : master_byte_word<BITS, J, 0>(w);
    return (uint8_t)((word >> (8 * (nb >> 1))) & 0xFFu);
  }
}

// all 32 sliced codes of a lane (index j*8 + e)
template <int BITS>
MATGPTQ_HD void master_decode_lane(const uint32_t* w, uint8_t (&codes)[32]) {
  MATGPTQ_UNROLL
  for (int e = 0; e < 8; e++) {
    codes[e] = master_code<BITS, 0>(w, e);
    codes[8 + e] = master_code<BITS, 1>(w, e);
    codes[16 + e] = master_code<BITS, 2>(w, e);
    codes[24 + e] = master_code<BITS, 3>(w, e);
  }
}

}  // namespace matgptq
