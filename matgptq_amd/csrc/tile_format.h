// What a GEMM kernel needs to know about the storage of a tile, as a policy type:
// how many words a lane holds, how to request them, how to turn octet J into the four raw
// fp16 pairs 1024 + c 2^p, and p.  Two storages: the pre-sliced b-bit layout of layout.h and the
// master-resident bit planes of master_layout.h (slice, rounding and saturation in registers).
#pragma once
#include "device_common.h"
#include "master_layout.h"

namespace matgptq {

template <int BITS, bool MASTER>
struct TileFormat;

template <int BITS>
struct TileFormat<BITS, false> {
  static constexpr int kWords = BITS;
  static constexpr uint32_t kTileBytes = (uint32_t)tile_words(BITS) * 4;
  static constexpr bool kScaledX = BITS != 8;  // some pair has p != 0
  static constexpr int raw_shift(int j, int i) { return Codec<BITS>::raw_shift(j, i); }
  using Consts = UnpackConsts<BITS>;
  // AUX: the cache policy of the loads (kAuxStream for data read once, 0 for data other workgroups read again)
  template <int AUX = kAuxStream>
  __device__ __forceinline__ static void load(BufRsrc rs, uint32_t tile_off, int lane, uint32_t (&w)[kWords]) {
    load_tile_words<BITS, AUX>(rs, tile_off, lane, w);
  }
  template <int J>
  __device__ __forceinline__ static void raw(const uint32_t (&w)[kWords], const Consts& k, uint32_t (&r)[4]) {
    raw_octet<BITS, J>(w, k, r);
  }
};

typedef uint32_t u32x3 __attribute__((ext_vector_type(3)));

template <int BITS>
struct TileFormat<BITS, true> {
  static constexpr int kWords = master_words(BITS);
  static constexpr uint32_t kTileBytes = kMasterTileWords * 4;
  static constexpr bool kScaledX = BITS <= 4;  // nibble form: pairs 1 and 3 carry p = 4
  static constexpr int raw_shift(int /*j*/, int i) { return BITS <= 4 ? ((i & 1) ? 4 : 0) : 0; }
  using Consts = UnpackConsts<4>;  // nibble masks and the magic word
  // one load per segment the bitwidth reads (S0: 12 bytes per lane, S1, S2: 4, S3: 12)
  template <int AUX = kAuxStream>
  __device__ __forceinline__ static void load(BufRsrc rs, uint32_t tile_off, int lane, uint32_t (&w)[kWords]) {
    const u32x3 a = __builtin_amdgcn_raw_buffer_load_b96(rs, lane * 12, tile_off, AUX);
    w[0] = a.x; w[1] = a.y; w[2] = a.z;
    if constexpr (BITS >= 3) w[3] = __builtin_amdgcn_raw_buffer_load_b32(rs, 768 + lane * 4, tile_off, AUX);
    if constexpr (BITS >= 4) w[4] = __builtin_amdgcn_raw_buffer_load_b32(rs, 1024 + lane * 4, tile_off, AUX);
    if constexpr (BITS >= 6) {
      const u32x3 c = __builtin_amdgcn_raw_buffer_load_b96(rs, 1280 + lane * 12, tile_off, AUX);
      w[5] = c.x; w[6] = c.y; w[7] = c.z;
    }
  }
  template <int J>
  __device__ __forceinline__ static void raw(const uint32_t (&w)[kWords], const Consts& k, uint32_t (&r)[4]) {
    if constexpr (BITS <= 4) {
      const uint32_t x = master_nibble_word<BITS, J>(w);
      const uint32_t x8 = x >> 8;
      r[0] = and_or(x, k.m[0], k.magic);
      r[1] = and_or(x, k.m[1], k.magic);
      r[2] = and_or(x8, k.m[0], k.magic);
      r[3] = and_or(x8, k.m[1], k.magic);
    } else {
      // pair i = (nibble index i, i + 4): bytes i/2 and i/2 + 2 of byte word i % 2
      const uint32_t w0 = master_byte_word<BITS, J, 0>(w), w1 = master_byte_word<BITS, J, 1>(w);
      const uint32_t fill = 0x64646464u;
      r[0] = __builtin_amdgcn_perm(fill, w0, 0x04020400u);
      r[1] = __builtin_amdgcn_perm(fill, w1, 0x04020400u);
      r[2] = __builtin_amdgcn_perm(fill, w0, 0x04030401u);
      r[3] = __builtin_amdgcn_perm(fill, w1, 0x04030401u);
    }
  }
};

// Octet J of a tile in either storage -> the 16 x 32 MFMA operand of dequantised weights (the
// arithmetic of dequant_octet / dequant_octet_bf16 in device_common.h on the format's raw pairs).
template <class Fmt, int BITS, int J, bool ZP>
__device__ __forceinline__ void dequant_octet_fmt(const uint32_t (&w)[Fmt::kWords], const typename Fmt::Consts& k,
                                                  half2v zrel, half2v scale, Frag& a) {
  uint32_t raw[4];
  Fmt::template raw<J>(w, k, raw);
  a.p[0] = dequant_pair<BITS, Fmt::raw_shift(J, 0), ZP>(raw[0], zrel, scale);
  a.p[1] = dequant_pair<BITS, Fmt::raw_shift(J, 1), ZP>(raw[1], zrel, scale);
  a.p[2] = dequant_pair<BITS, Fmt::raw_shift(J, 2), ZP>(raw[2], zrel, scale);
  a.p[3] = dequant_pair<BITS, Fmt::raw_shift(J, 3), ZP>(raw[3], zrel, scale);
}
template <class Fmt, int BITS, int J>
__device__ __forceinline__ void dequant_octet_bf16_fmt(const uint32_t (&w)[Fmt::kWords], const typename Fmt::Consts& k,
                                                       float sm, float sz, Frag& a) {
  uint32_t raw[4];
  Fmt::template raw<J>(w, k, raw);
  a.u[0] = dequant_pair_bf16<BITS, Fmt::raw_shift(J, 0)>(raw[0], sm, sz);
  a.u[1] = dequant_pair_bf16<BITS, Fmt::raw_shift(J, 1)>(raw[1], sm, sz);
  a.u[2] = dequant_pair_bf16<BITS, Fmt::raw_shift(J, 2)>(raw[2], sm, sz);
  a.u[3] = dequant_pair_bf16<BITS, Fmt::raw_shift(J, 3)>(raw[3], sm, sz);
}

// Number of load instructions TileFormat::load issues for one tile.
constexpr int master_load_count(int bits) { return bits == 2 ? 1 : bits == 3 ? 2 : bits == 4 ? 3 : 4; }

}  // namespace matgptq
