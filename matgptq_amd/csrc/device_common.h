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

// ---- bfloat16 storage (activations, scales, zeros, output when the BF16 flag is set) ----
// The decode-regime kernels compute in fp16 operands / fp32 accumulators either way; bf16 values
// are converted where they enter and leave.  bf16 -> fp16 is exact inside fp16's normal range
// (8 significant bits into 11); magnitudes above 65504 saturate to +-65504.  The prefill kernel
// multiplies bf16 by bf16 on the matrix cores (no conversion of the activations, no saturation).
#ifndef MATGPTQ_BF16
#define MATGPTQ_BF16 0
#endif
constexpr bool kBf16 = MATGPTQ_BF16 != 0;

__device__ __forceinline__ float bf16_bits_to_float(uint32_t b) { return __uint_as_float(b << 16); }

// round to nearest even; NaN stays NaN
__device__ __forceinline__ uint32_t float_to_bf16_bits(float f) {
  const uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0u;
  return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

// 16-bit storage element (fp16 or bf16, by MATGPTQ_BF16) -> float, and float -> storage
__device__ __forceinline__ float storage_to_float(uint16_t b) {
  if constexpr (kBf16) return bf16_bits_to_float(b);
  return (float)__builtin_bit_cast(_Float16, b);
}
__device__ __forceinline__ uint16_t float_to_storage(float f) {
  if constexpr (kBf16) return (uint16_t)float_to_bf16_bits(f);
  return __builtin_bit_cast(uint16_t, (_Float16)f);
}
__device__ __forceinline__ _Float16 storage_to_half(uint16_t b) {
  if constexpr (kBf16) return (_Float16)bf16_bits_to_float(b);
  return __builtin_bit_cast(_Float16, b);
}

// two bf16 in one word -> two fp16 (saturating)
__device__ __forceinline__ half2v bf16x2_to_half2(uint32_t w) {
  float lo = __uint_as_float(w << 16), hi = __uint_as_float(w & 0xffff0000u);
  lo = __builtin_fminf(__builtin_fmaxf(lo, -65504.0f), 65504.0f);
  hi = __builtin_fminf(__builtin_fmaxf(hi, -65504.0f), 65504.0f);
  return half2v{(_Float16)lo, (_Float16)hi};
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

// eight stored activations (one 16-byte chunk) -> eight fp16
__device__ __forceinline__ half8 storage8_to_half8(half8 raw) {
  if constexpr (kBf16) {
    Frag in, out;
    in.h = raw;
#pragma unroll
    for (int i = 0; i < 4; i++) out.p[i] = bf16x2_to_half2(in.u[i]);
    return out.h;
  }
  return raw;
}

// (x & mask) | orv.  The compiler folds this into one v_and_or_b32 when neither constant
// is a literal: a VOP3 encoding of this target takes no literal and one scalar operand.
// `opaque_*` hide a constant's value from the optimiser (no instruction is emitted), so the
// mask stays in an SGPR and the OR-ed word in a VGPR.  The instruction itself is chosen by
// the compiler, which keeps its hazard bookkeeping (VALU result -> MFMA operand) intact.
__device__ __forceinline__ uint32_t opaque_sgpr(uint32_t v) {
  asm("" : "+s"(v));
  return v;
}
__device__ __forceinline__ uint32_t opaque_vgpr(uint32_t v) {
  asm("" : "+v"(v));
  return v;
}
__device__ __forceinline__ uint32_t and_or(uint32_t x, uint32_t mask, uint32_t orv) {
  return (x & mask) | orv;
}

// The constants of the unpack sequence, made opaque once per kernel.
template <int BITS>
struct UnpackConsts {
  uint32_t magic;  // VGPR: two fp16 1024.0
  uint32_t m[4];   // SGPRs: field masks
  __device__ __forceinline__ UnpackConsts() {
    magic = opaque_vgpr(kMagic);
    if constexpr (BITS == 2) {
      m[0] = opaque_sgpr(0x00030003u); m[1] = opaque_sgpr(0x000C000Cu); m[2] = opaque_sgpr(0x00300030u);
    } else if constexpr (BITS == 6) {
      m[0] = opaque_sgpr(0x00030003u); m[1] = opaque_sgpr(0x00300030u);
      m[2] = opaque_sgpr(0x003C003Cu); m[3] = opaque_sgpr(0x03C003C0u);
    } else if constexpr (BITS == 3) {
      m[0] = opaque_sgpr(0x000F000Fu); m[1] = opaque_sgpr(0x00F000F0u); m[2] = opaque_sgpr(0x44444444u);
    } else {
      m[0] = opaque_sgpr(0x000F000Fu); m[1] = opaque_sgpr(0x00F000F0u); m[2] = 0;
    }
  }
};

// Device form of Codec<BITS>::decode_octet (same results, fewer instructions):
// the four raw pairs 1024 + c * 2^p of octet J.
template <int BITS, int J>
__device__ __forceinline__ void raw_octet(const uint32_t (&w)[BITS], const UnpackConsts<BITS>& k,
                                          uint32_t (&r)[4]) {
  if constexpr (BITS == 4 || BITS == 3) {
    uint32_t x;
    if constexpr (BITS == 4) {
      x = w[J];
    } else {
      const uint32_t lo = (w[J >> 1] >> (2 * (J & 1))) & 0x33333333u;
      const uint32_t c = w[2];
      const uint32_t cs = J == 0 ? (c << 2) : J == 1 ? (c << 1) : J == 2 ? c : (c >> 1);
      x = and_or(cs, k.m[2], lo);
    }
    const uint32_t x8 = x >> 8;
    r[0] = and_or(x, k.m[0], k.magic);
    r[1] = and_or(x, k.m[1], k.magic);
    r[2] = and_or(x8, k.m[0], k.magic);
    r[3] = and_or(x8, k.m[1], k.magic);
  } else if constexpr (BITS == 2) {
    const uint32_t x = w[J >> 1];
    const uint32_t x6 = x >> 6;
    if constexpr ((J & 1) == 0) {
      r[0] = and_or(x, k.m[0], k.magic);
      r[1] = and_or(x, k.m[1], k.magic);
      r[2] = and_or(x, k.m[2], k.magic);
      r[3] = and_or(x6, k.m[0], k.magic);
    } else {
      const uint32_t x12 = x >> 12;
      r[0] = and_or(x6, k.m[1], k.magic);
      r[1] = and_or(x6, k.m[2], k.magic);
      r[2] = and_or(x12, k.m[0], k.magic);
      r[3] = and_or(x12, k.m[1], k.magic);
    }
  } else if constexpr (BITS == 6) {
    // high nibbles shifted to bits 2..5 of their fields once per word (<< 2 for pairs 0, 1; >> 6 for
    // pairs 2, 3, whose nibbles sit 8 bits higher); a pair is then two v_and_or_b32: the low bits
    // over the magic word, the high nibble over that (their bit ranges are disjoint)
    const uint32_t hs = w[J] << 2, hs6 = w[J] >> 6;
    const uint32_t l = (J & 1) ? (w[4 + (J >> 1)] >> 8) : w[4 + (J >> 1)];
    const uint32_t l2 = l >> 2;
    // (the inner result is hidden from the optimiser, which would otherwise regroup the two
    // v_and_or_b32 of a pair into two v_and_b32 and a v_or3_b32)
    r[0] = and_or(hs, k.m[2], opaque_vgpr(and_or(l, k.m[0], k.magic)));
    r[1] = and_or(hs, k.m[3], opaque_vgpr(and_or(l, k.m[1], k.magic)));
    r[2] = and_or(hs6, k.m[2], opaque_vgpr(and_or(l2, k.m[0], k.magic)));
    r[3] = and_or(hs6, k.m[3], opaque_vgpr(and_or(l2, k.m[1], k.magic)));
  } else {
    // bytes: pair 2d = (byte0, byte2) of word 2J+d, pair 2d+1 = (byte1, byte3)
    const uint32_t fill = 0x64646464u;
    r[0] = __builtin_amdgcn_perm(fill, w[2 * J], 0x04020400u);
    r[1] = __builtin_amdgcn_perm(fill, w[2 * J], 0x04030401u);
    r[2] = __builtin_amdgcn_perm(fill, w[2 * J + 1], 0x04020400u);
    r[3] = __builtin_amdgcn_perm(fill, w[2 * J + 1], 0x04030401u);
  }
}

// Octet j of a lane -> MFMA operand holding (c - 2^(b-1)) for its eight codes.
template <int BITS, int J>
__device__ __forceinline__ void centred_octet(const uint32_t (&w)[BITS], const UnpackConsts<BITS>& k,
                                              Frag& a) {
  uint32_t raw[4];
  raw_octet<BITS, J>(w, k, raw);
  constexpr int c = Codec<BITS>::kCentre;
  a.p[0] = centre_raw<Codec<BITS>::raw_shift(J, 0)>(raw[0], c);
  a.p[1] = centre_raw<Codec<BITS>::raw_shift(J, 1)>(raw[1], c);
  a.p[2] = centre_raw<Codec<BITS>::raw_shift(J, 2)>(raw[2], c);
  a.p[3] = centre_raw<Codec<BITS>::raw_shift(J, 3)>(raw[3], c);
}

// One raw pair -> two weights.  u = c - 2^(b-1) is exact.
//   symmetric, fp16 storage:  w = u * (scale * m),  m = 2^(8-b) (a power of two: one rounding,
//     the value the reference's dequantize() gives);
//   zero point, fp16 storage: w = fma(u, scale * m, -(scale * zrel)),  zrel = zero - 128: two
//     instructions per pair instead of three.  scale * zrel is rounded to fp16 before the fma,
//     so w can differ from dequantize()'s  fp16(scale * fp16(m u - zrel))  by one rounding of a
//     term no larger than 128 scale: at most scale / 16, less than the rounding error of w
//     itself (the dense dequantize_matgptq operator keeps the reference's exact sequence);
//   bf16 storage: a bf16 scale can lie far below fp16's normal range, so the caller passes
//     scale * 2^8 and zrel * 2^-8 and  v = m u 2^-8 - zrel 2^-8  is formed exactly and
//     multiplied by the scale (the symmetric form takes the same route with zrel = 0).
// `a`, `b`: (scale * m, scale * zrel) for fp16 storage with zero points, (scale', zrel') else.
template <int BITS, int P, bool ZP>
__device__ __forceinline__ half2v dequant_pair(uint32_t raw, half2v b, half2v a) {
  const half2v u = centre_raw<P>(raw, Codec<BITS>::kCentre);
  if constexpr (kBf16) {
    constexpr float m = (float)(1 << (8 - BITS)) / 256.0f;
    const half2v v = __builtin_elementwise_fma(u, h2_splat(m), -b);
    return v * a;
  } else if constexpr (ZP) {
    return __builtin_elementwise_fma(u, a, -b);
  } else {
    return u * a;
  }
}

template <int BITS, int J, bool ZP>
__device__ __forceinline__ void dequant_octet(const uint32_t (&w)[BITS], const UnpackConsts<BITS>& k,
                                              half2v zrel, half2v scale, Frag& a) {
  uint32_t raw[4];
  raw_octet<BITS, J>(w, k, raw);
  a.p[0] = dequant_pair<BITS, Codec<BITS>::raw_shift(J, 0), ZP>(raw[0], zrel, scale);
  a.p[1] = dequant_pair<BITS, Codec<BITS>::raw_shift(J, 1), ZP>(raw[1], zrel, scale);
  a.p[2] = dequant_pair<BITS, Codec<BITS>::raw_shift(J, 2), ZP>(raw[2], zrel, scale);
  a.p[3] = dequant_pair<BITS, Codec<BITS>::raw_shift(J, 3), ZP>(raw[3], zrel, scale);
}

// bf16 storage on the matrix cores' bf16 path (the prefill kernel): the weight is formed in fp32,
//   w = bf16(fma(u, scale m, -(scale zrel))),  `sm` = scale m, `sz` = scale zrel,
// one fused conversion and multiply-add per element and one packed conversion per pair.  u (8 bits),
// a bf16 scale (8 bits) and an integer zero point (8 bits) make both products and their difference
// exact in fp32, so w is scale (m c - zero) rounded once: the value dequantize() gives on bfloat16
// tensors whenever m c - zero is itself a bfloat16 (always, for integer zero points).
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float2v __attribute__((ext_vector_type(2)));

// The centring of the raw pair rides in the same fused multiply-add: with r = 1024 + c 2^P,
//   scale (m c - zero) = r (sm 2^-P) - (sz + (1024 2^-P + centre) sm),
// both constants per (row, group, P), formed once and exact in fp32 as long as the integer
// 255 (128 + m (1024 2^-P + centre)) stays below 2^24 (every pair but the P = 0 pairs of 2-bit codes,
// which keep the separate centring step).
template <int BITS, int P>
__device__ __forceinline__ uint32_t dequant_pair_bf16(uint32_t raw, float sm, float sz) {
  constexpr int kM = 1 << (8 - BITS);
  constexpr bool kFold = 255ll * (128 + (long long)kM * ((1024 >> P) + Codec<BITS>::kCentre)) < (1ll << 24) && (1024 >> P) << P == 1024;
  // (symmetric layers pass an opaque zero as `sz`: the fused form is one instruction per element,
  // a conversion followed by a multiplication two)
  if constexpr (kFold) {
    const half2v r = h2_from_bits(raw);
    const float sp = sm * (1.0f / (float)(1 << P));
    const float zp = __builtin_fmaf((float)((1024 >> P) + Codec<BITS>::kCentre), sm, sz);
    const float2v w = {__builtin_fmaf((float)r.x, sp, -zp), __builtin_fmaf((float)r.y, sp, -zp)};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(w, bf16x2));
  } else {
    const half2v u = centre_raw<P>(raw, Codec<BITS>::kCentre);
    const float2v w = {__builtin_fmaf((float)u.x, sm, -sz), __builtin_fmaf((float)u.y, sm, -sz)};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(w, bf16x2));
  }
}

template <int BITS, int J>
__device__ __forceinline__ void dequant_octet_bf16(const uint32_t (&w)[BITS], const UnpackConsts<BITS>& k,
                                                   float sm, float sz, Frag& a) {
  uint32_t raw[4];
  raw_octet<BITS, J>(w, k, raw);
  a.u[0] = dequant_pair_bf16<BITS, Codec<BITS>::raw_shift(J, 0)>(raw[0], sm, sz);
  a.u[1] = dequant_pair_bf16<BITS, Codec<BITS>::raw_shift(J, 1)>(raw[1], sm, sz);
  a.u[2] = dequant_pair_bf16<BITS, Codec<BITS>::raw_shift(J, 2)>(raw[2], sm, sz);
  a.u[3] = dequant_pair_bf16<BITS, Codec<BITS>::raw_shift(J, 3)>(raw[3], sm, sz);
}

// Buffer resources: a 128-bit scalar descriptor (base, byte size) lets every load
// take its wave-uniform part from an SGPR and its per-lane part from one 32-bit
// VGPR, so a stream of tile loads needs no vector address arithmetic; reads past
// the size return zero.  Offsets are 32-bit: a tensor must stay below 4 GiB.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __amdgpu_buffer_rsrc_t BufRsrc;
constexpr int kAuxStream = 2;  // "nt": data that is read once

__device__ __forceinline__ BufRsrc make_rsrc(const void* p, uint32_t bytes) {
  // word 3 = 0x00020000: untyped 32-bit data format of this target's buffer descriptors
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

// Number of load instructions load_tile_words issues for one tile (kernels that count their
// loads in flight by hand use it).
constexpr int tile_load_count(int bits) { return bits == 3 || bits == 6 || bits == 8 ? 2 : 1; }

// Loads the BITS words of `lane` from the tile that starts `tile_bytes` into the buffer
// (wave-uniform), one load per segment.  AUX = kAuxStream for data read once (decode),
// 0 for data other workgroups read again (prefill).
template <int BITS, int AUX = kAuxStream>
__device__ __forceinline__ void load_tile_words(BufRsrc rs, uint32_t tile_bytes, int lane,
                                                uint32_t (&w)[BITS]) {
  constexpr int kAuxStream = AUX;  // shadows the global constant below on purpose
  if constexpr (BITS == 2) {
    const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rs, lane * 8, tile_bytes, kAuxStream);
    w[0] = v.x; w[1] = v.y;
  } else if constexpr (BITS == 3) {
    const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rs, lane * 8, tile_bytes, kAuxStream);
    w[0] = v.x; w[1] = v.y;
    w[2] = __builtin_amdgcn_raw_buffer_load_b32(rs, 512 + lane * 4, tile_bytes, kAuxStream);
  } else if constexpr (BITS == 4) {
    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rs, lane * 16, tile_bytes, kAuxStream);
    w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
  } else if constexpr (BITS == 6) {
    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rs, lane * 16, tile_bytes, kAuxStream);
    w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
    const u32x2 l = __builtin_amdgcn_raw_buffer_load_b64(rs, 1024 + lane * 8, tile_bytes, kAuxStream);
    w[4] = l.x; w[5] = l.y;
  } else {
    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rs, lane * 16, tile_bytes, kAuxStream);
    w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
    const u32x4 l = __builtin_amdgcn_raw_buffer_load_b128(rs, 1024 + lane * 16, tile_bytes, kAuxStream);
    w[4] = l.x; w[5] = l.y; w[6] = l.z; w[7] = l.w;
  }
}

// Same from a plain pointer (load-time kernels).
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

// Prefill with a tail of narrower tiles: how many 256-row weight tiles (of `row_blocks / 16` whole
// ones) the 128 x 256 workgroups take before the 128 x 128 workgroups take the remaining rows -
// the whole rounds of 512 resident workgroups (two per CU), in whole columns of `m_tiles`
// activation tiles.
inline int prefill_tail_big_tiles(int row_blocks, int m_tiles) {
  const int n_tiles = row_blocks / 16;
  const int per_round = 512 / m_tiles;  // weight tiles one round covers
  if (per_round == 0) return n_tiles;
  return n_tiles / per_round * per_round;
}

}  // namespace matgptq
