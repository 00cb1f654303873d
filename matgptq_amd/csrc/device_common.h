// Device-side helpers shared by the gfx950 kernels: vector types, the raw ->
// fp16 operand conversion, argument blocks.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "layout.h"

namespace matgptq {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));

union Frag {  // one MFMA 16x16x32 f16 operand: eight halves per lane
  half8 h;
  half2v p[4];
  uint32_t u[4];
  uint4 v;
};

union H2 {
  half2v h;
  uint32_t u;
};

union H4 {  // four fp16 loaded as one 8-byte word
  uint2 v;
  _Float16 h[4];
};

__device__ __forceinline__ half2v h2_splat(float f) {
  half2v r = {(_Float16)f, (_Float16)f};
  return r;
}

__device__ __forceinline__ half2v h2_from_bits(uint32_t u) {
  H2 t;
  t.u = u;
  return t.h;
}

// Raw pair (1024 + c * 2^p, twice) -> (c - centre, twice), exactly.
// (1024 + c 2^p) * 2^-p = 1024 * 2^-p + c is exact in fp16 for every p used
// (p <= 8 and c < 2^(10-p)); so is the subtraction of the integer constant.
template <int P>
__device__ __forceinline__ half2v centre_raw(uint32_t raw, int centre) {
  const half2v v = h2_from_bits(raw);
  if constexpr (P == 0) {
    return v - h2_splat(1024.0f + (float)centre);
  } else {
    const float inv = 1.0f / (float)(1 << P);
    return __builtin_elementwise_fma(v, h2_splat(inv), h2_splat(-(1024.0f * inv + (float)centre)));
  }
}

// Octet j of a lane -> MFMA operand holding (c - 2^(b-1)) for its eight codes.
template <int BITS, int J>
__device__ __forceinline__ void centred_octet(const uint32_t (&w)[BITS], Frag& a) {
  uint32_t raw[4];
  Codec<BITS>::decode_octet(w, J, raw);
  constexpr int c = Codec<BITS>::kCentre;
  a.p[0] = centre_raw<Codec<BITS>::raw_shift(J, 0)>(raw[0], c);
  a.p[1] = centre_raw<Codec<BITS>::raw_shift(J, 1)>(raw[1], c);
  a.p[2] = centre_raw<Codec<BITS>::raw_shift(J, 2)>(raw[2], c);
  a.p[3] = centre_raw<Codec<BITS>::raw_shift(J, 3)>(raw[3], c);
}

// Loads the BITS words of `lane` from a tile with one load per segment.
template <int BITS>
__device__ __forceinline__ void load_tile_words(const uint32_t* __restrict__ tile, int lane,
                                                uint32_t (&w)[BITS]) {
  if constexpr (BITS == 2) {
    const uint2 v = *reinterpret_cast<const uint2*>(tile + lane * 2);
    w[0] = v.x; w[1] = v.y;
  } else if constexpr (BITS == 3) {
    const uint2 v = *reinterpret_cast<const uint2*>(tile + lane * 2);
    w[0] = v.x; w[1] = v.y;
    w[2] = tile[128 + lane];
  } else if constexpr (BITS == 4) {
    const uint4 v = *reinterpret_cast<const uint4*>(tile + lane * 4);
    w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
  } else if constexpr (BITS == 6) {
    const uint4 v = *reinterpret_cast<const uint4*>(tile + lane * 4);
    w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
    const uint2 l = *reinterpret_cast<const uint2*>(tile + 256 + lane * 2);
    w[4] = l.x; w[5] = l.y;
  } else {
    const uint4 v = *reinterpret_cast<const uint4*>(tile + lane * 4);
    w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
    const uint4 l = *reinterpret_cast<const uint4*>(tile + 256 + lane * 4);
    w[4] = l.x; w[5] = l.y; w[6] = l.z; w[7] = l.w;
  }
}

struct GemmArgs {
  const uint32_t* packed;   // tiled codes
  const uint16_t* scales;   // [N/16][G][16] fp16 bits
  const uint16_t* zeros;    // same layout, or nullptr (all 128)
  const uint16_t* x;        // [M, K] fp16 bits
  uint16_t* y;              // [M, N] fp16 bits
  int N, K, M;
  int G;                    // groups per row (1 for group_size -1)
  int k_tiles;              // K / 128
  int row_blocks;           // N / 16
};

}  // namespace matgptq
