// Host-side packers: sliced (or master) uint8 codes -> tiled gfx950 layout, the
// inverse, and the scale/zero reorder.  Plain C++ (no HIP), OpenMP over row blocks.
// Counterpart of the reference's CPU repack (inference_lib/matgptq_cuda/csrc/utils.cpp:22-217,
// bindings.cpp:43-142), with its own layout (see layout.h).
#include <cstring>

#include "../../include/matgptq_abi.h"
#include "layout.h"
#include "master_layout.h"

namespace matgptq {

int check_problem(int bits, int group_size, int64_t N, int64_t K) {
  if (!valid_bits(bits)) return MATGPTQ_EBITS;
  if (N <= 0 || N % kTileRows != 0 || !valid_k(K)) return MATGPTQ_ESHAPE;
  if (!valid_group(group_size)) return MATGPTQ_EGROUP;
  if (group_size != -1 && K % group_size != 0) return MATGPTQ_EGROUP;
  return MATGPTQ_OK;
}

template <int BITS>
static void pack_impl(const uint8_t* codes, int64_t N, int64_t K, bool slice, uint32_t* out) {
  const int64_t row_blocks = N / kTileRows, k_blocks = K / kTileCols;
#pragma omp parallel for schedule(static)
  for (int64_t rb = 0; rb < row_blocks; rb++) {
    for (int64_t kb = 0; kb < k_blocks; kb++) {
      uint32_t* tile = out + (rb * k_blocks + kb) * tile_words(BITS);
      for (int lane = 0; lane < kLanes; lane++) {
        const int r = lane % 16, q = lane / 16;
        const uint8_t* row = codes + (rb * kTileRows + r) * K + kb * kTileCols;
        uint8_t c[32];
        for (int j = 0; j < 4; j++)
          for (int e = 0; e < 8; e++) {
            const uint8_t v = row[j * 32 + q * 8 + e];
            c[j * 8 + e] = slice ? slice_code(v, BITS) : v;
          }
        uint32_t w[BITS];
        Codec<BITS>::encode_lane(c, w);
        for (int i = 0; i < BITS; i++) tile[word_offset(BITS, lane, i)] = w[i];
      }
    }
  }
  if (K % kTileCols != 0) {  // the last 64 columns, one bitstream per row
    uint32_t* tail = out + row_blocks * k_blocks * tile_words(BITS);
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; n++) {
      uint8_t c[kTailCols];
      for (int k = 0; k < kTailCols; k++) {
        const uint8_t v = codes[n * K + k_blocks * kTileCols + k];
        c[k] = slice ? slice_code(v, BITS) : v;
      }
      tail_encode_row(c, BITS, tail + n * tail_row_words(BITS));
    }
  }
}

template <int BITS>
static void unpack_impl(const uint32_t* packed, int64_t N, int64_t K, uint8_t* codes) {
  const int64_t row_blocks = N / kTileRows, k_blocks = K / kTileCols;
#pragma omp parallel for schedule(static)
  for (int64_t rb = 0; rb < row_blocks; rb++) {
    for (int64_t kb = 0; kb < k_blocks; kb++) {
      const uint32_t* tile = packed + (rb * k_blocks + kb) * tile_words(BITS);
      for (int lane = 0; lane < kLanes; lane++) {
        const int r = lane % 16, q = lane / 16;
        uint8_t* row = codes + (rb * kTileRows + r) * K + kb * kTileCols;
        uint32_t w[BITS];
        for (int i = 0; i < BITS; i++) w[i] = tile[word_offset(BITS, lane, i)];
        for (int j = 0; j < 4; j++) {
          uint32_t raw[4];
          Codec<BITS>::decode_octet(w, j, raw);
          for (int e = 0; e < 8; e++) row[j * 32 + q * 8 + e] = code_from_raw<BITS>(raw, j, e);
        }
      }
    }
  }
  if (K % kTileCols != 0) {
    const uint32_t* tail = packed + row_blocks * k_blocks * tile_words(BITS);
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; n++)
      for (int k = 0; k < kTailCols; k++)
        codes[n * K + k_blocks * kTileCols + k] = (uint8_t)tail_code(tail + n * tail_row_words(BITS), BITS, k);
  }
}

template <int BITS>
static void master_slice_impl(const uint32_t* planes, int64_t N, int64_t K, uint8_t* codes) {
  const int64_t row_blocks = N / kTileRows, k_blocks = K / kTileCols;
#pragma omp parallel for schedule(static)
  for (int64_t rb = 0; rb < row_blocks; rb++) {
    for (int64_t kb = 0; kb < k_blocks; kb++) {
      const uint32_t* tile = planes + (rb * k_blocks + kb) * kMasterTileWords;
      for (int lane = 0; lane < kLanes; lane++) {
        uint32_t w[8];
        for (int i = 0; i < 8; i++) w[i] = i < master_words(BITS) ? tile[master_word_offset(lane, i)] : 0u;
        uint8_t c[32];
        master_decode_lane<BITS>(w, c);
        uint8_t* row = codes + (rb * kTileRows + lane % 16) * K + kb * kTileCols + (lane / 16) * 8;
        for (int j = 0; j < 4; j++)
          for (int e = 0; e < 8; e++) row[j * 32 + e] = c[j * 8 + e];
      }
    }
  }
}

}  // namespace matgptq

using namespace matgptq;

extern "C" {

size_t matgptq_packed_words(int bitwidth, int64_t N, int64_t K) {
  if (!valid_bits(bitwidth) || N <= 0 || K <= 0) return 0;
  return (size_t)bitwidth * (size_t)N * (size_t)K / 32;
}

int matgptq_pack_host(const uint8_t* codes_host, int64_t N, int64_t K, int bitwidth,
                      int slice_from_master, uint32_t* out_host) {
  if (int e = check_problem(bitwidth, -1, N, K)) return e;
  if (!codes_host || !out_host) return MATGPTQ_ENULL;
  const bool s = slice_from_master != 0;
  switch (bitwidth) {
    case 2: pack_impl<2>(codes_host, N, K, s, out_host); break;
    case 3: pack_impl<3>(codes_host, N, K, s, out_host); break;
    case 4: pack_impl<4>(codes_host, N, K, s, out_host); break;
    case 6: pack_impl<6>(codes_host, N, K, s, out_host); break;
    case 8: pack_impl<8>(codes_host, N, K, s, out_host); break;
  }
  return MATGPTQ_OK;
}

int matgptq_unpack_host(const uint32_t* packed_host, int64_t N, int64_t K, int bitwidth,
                        uint8_t* codes_host) {
  if (int e = check_problem(bitwidth, -1, N, K)) return e;
  if (!packed_host || !codes_host) return MATGPTQ_ENULL;
  switch (bitwidth) {
    case 2: unpack_impl<2>(packed_host, N, K, codes_host); break;
    case 3: unpack_impl<3>(packed_host, N, K, codes_host); break;
    case 4: unpack_impl<4>(packed_host, N, K, codes_host); break;
    case 6: unpack_impl<6>(packed_host, N, K, codes_host); break;
    case 8: unpack_impl<8>(packed_host, N, K, codes_host); break;
  }
  return MATGPTQ_OK;
}

size_t matgptq_master_words(int64_t N, int64_t K) {
  if (N <= 0 || K <= 0 || N % kTileRows != 0 || K % kTileCols != 0) return 0;
  return (size_t)N * (size_t)K / 4;
}

int matgptq_pack_master_host(const uint8_t* codes_host, int64_t N, int64_t K, uint32_t* out_host) {
  if (int e = check_problem(8, -1, N, K)) return e;
  if (K % kTileCols != 0) return MATGPTQ_ESHAPE;  // the bit planes have whole tiles only
  if (!codes_host || !out_host) return MATGPTQ_ENULL;
  const int64_t row_blocks = N / kTileRows, k_blocks = K / kTileCols;
#pragma omp parallel for schedule(static)
  for (int64_t rb = 0; rb < row_blocks; rb++)
    for (int64_t kb = 0; kb < k_blocks; kb++) {
      uint32_t* tile = out_host + (rb * k_blocks + kb) * kMasterTileWords;
      for (int lane = 0; lane < kLanes; lane++) {
        const uint8_t* row = codes_host + (rb * kTileRows + lane % 16) * K + kb * kTileCols + (lane / 16) * 8;
        uint8_t c[32];
        for (int j = 0; j < 4; j++)
          for (int e = 0; e < 8; e++) c[j * 8 + e] = row[j * 32 + e];
        uint32_t w[8];
        master_encode_lane(c, w);
        for (int i = 0; i < 8; i++) tile[master_word_offset(lane, i)] = w[i];
      }
    }
  return MATGPTQ_OK;
}

int matgptq_unpack_master_host(const uint32_t* planes_host, int64_t N, int64_t K, int bitwidth,
                               uint8_t* codes_host) {
  if (int e = check_problem(bitwidth, -1, N, K)) return e;
  if (K % kTileCols != 0) return MATGPTQ_ESHAPE;
  if (!planes_host || !codes_host) return MATGPTQ_ENULL;
  switch (bitwidth) {
    case 2: master_slice_impl<2>(planes_host, N, K, codes_host); break;
    case 3: master_slice_impl<3>(planes_host, N, K, codes_host); break;
    case 4: master_slice_impl<4>(planes_host, N, K, codes_host); break;
    case 6: master_slice_impl<6>(planes_host, N, K, codes_host); break;
    case 8: master_slice_impl<8>(planes_host, N, K, codes_host); break;
  }
  return MATGPTQ_OK;
}

int matgptq_reorder_scales_host(const uint16_t* in_host, int64_t N, int64_t K, int group_size,
                                uint16_t* out_host) {
  if (int e = check_problem(8, group_size, N, K)) return e;
  if (!in_host || !out_host) return MATGPTQ_ENULL;
  const int64_t G = group_size == -1 ? 1 : K / group_size;
  const int64_t row_blocks = N / kTileRows;
#pragma omp parallel for schedule(static)
  for (int64_t rb = 0; rb < row_blocks; rb++)
    for (int64_t g = 0; g < G; g++)
      for (int r = 0; r < kTileRows; r++)
        out_host[(rb * G + g) * kTileRows + r] = in_host[(rb * kTileRows + r) * G + g];
  return MATGPTQ_OK;
}

}  // extern "C"
