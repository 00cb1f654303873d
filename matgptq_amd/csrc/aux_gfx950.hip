// Load-time and debug kernels: slice, pack, unpack, scale reorder, dense dequantise.
// They replace the reference's host round trip for tensors that already live in HBM
// (inference_lib/matgptq_cuda/csrc/bindings.cpp:63-83,99-141) and give tests a
// device-side view of the packed codes.  All are byte/integer work, HBM-bound.
#include "device_common.h"
#include "master_layout.h"

namespace matgptq {

namespace {

// One thread = one lane slot of one tile: 32 codes in, BITS words out.
template <int BITS>
__global__ void __launch_bounds__(256)
pack_kernel(const uint8_t* __restrict__ codes, uint32_t* __restrict__ out, int k_tiles,
            int64_t K, int64_t total_slots, int slice) {
  const int64_t slot = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (slot >= total_slots) return;
  const int lane = (int)(slot & 63);
  const int64_t tile = slot >> 6;
  const int64_t rb = tile / k_tiles, kb = tile - rb * k_tiles;
  const int r = lane & 15, q = lane >> 4;
  const uint8_t* row = codes + (rb * 16 + r) * K + kb * 128 + q * 8;
  uint8_t c[32];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const uint2 v = *reinterpret_cast<const uint2*>(row + j * 32);
    const uint32_t lo = v.x, hi = v.y;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      c[j * 8 + e] = (uint8_t)(lo >> (8 * e));
      c[j * 8 + 4 + e] = (uint8_t)(hi >> (8 * e));
    }
  }
  if (slice) {
#pragma unroll
    for (int i = 0; i < 32; i++) c[i] = slice_code(c[i], BITS);
  }
  uint32_t w[BITS];
  Codec<BITS>::encode_lane(c, w);
  uint32_t* t = out + tile * tile_words(BITS);
#pragma unroll
  for (int i = 0; i < BITS; i++) t[word_offset(BITS, lane, i)] = w[i];
}

template <int BITS>
__global__ void __launch_bounds__(256)
unpack_kernel(const uint32_t* __restrict__ packed, uint8_t* __restrict__ codes, int k_tiles,
              int64_t K, int64_t total_slots) {
  const int64_t slot = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (slot >= total_slots) return;
  const int lane = (int)(slot & 63);
  const int64_t tile = slot >> 6;
  const int64_t rb = tile / k_tiles, kb = tile - rb * k_tiles;
  const int r = lane & 15, q = lane >> 4;
  const UnpackConsts<BITS> kc_unpack;
  uint32_t w[BITS];
  load_tile_words<BITS>(packed + tile * tile_words(BITS), lane, w);
  uint8_t* row = codes + (rb * 16 + r) * K + kb * 128 + q * 8;
  auto emit = [&](auto jtag) {
    constexpr int J = decltype(jtag)::value;
    uint32_t raw[4];
    raw_octet<BITS, J>(w, kc_unpack, raw);
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      lo |= (uint32_t)code_from_raw<BITS>(raw, J, e) << (8 * e);
      hi |= (uint32_t)code_from_raw<BITS>(raw, J, 4 + e) << (8 * e);
    }
    *reinterpret_cast<uint2*>(row + J * 32) = make_uint2(lo, hi);
  };
  emit(std::integral_constant<int, 0>{});
  emit(std::integral_constant<int, 1>{});
  emit(std::integral_constant<int, 2>{});
  emit(std::integral_constant<int, 3>{});
}

__global__ void __launch_bounds__(256)
slice_kernel(const uint8_t* __restrict__ in, uint8_t* __restrict__ out, int64_t count, int bits) {
  const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i + 4 <= count && ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 3) == 0) {
    const uint32_t v = *reinterpret_cast<const uint32_t*>(in + i);
    uint32_t o = 0;
#pragma unroll
    for (int e = 0; e < 4; e++) o |= (uint32_t)slice_code((uint8_t)(v >> (8 * e)), bits) << (8 * e);
    *reinterpret_cast<uint32_t*>(out + i) = o;
  } else {
    for (int64_t e = i; e < count && e < i + 4; e++) out[e] = slice_code(in[e], bits);
  }
}

// [N, G] -> [N/16][G][16]
__global__ void __launch_bounds__(256)
reorder_kernel(const uint16_t* __restrict__ in, uint16_t* __restrict__ out, int64_t G,
               int64_t total) {
  const int64_t o = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (o >= total) return;
  const int r = (int)(o & 15);
  const int64_t t = o >> 4;
  const int64_t rb = t / G, g = t - rb * G;
  out[o] = in[(rb * 16 + r) * G + g];
}

// Dense W[N,K] = fp16(scale * fp16((c << (8-b)) - zero)), one lane slot per thread.
template <int BITS>
__global__ void __launch_bounds__(256)
dequant_kernel(const uint32_t* __restrict__ packed, const uint16_t* __restrict__ scales,
               const uint16_t* __restrict__ zeros, uint16_t* __restrict__ w_out, int k_tiles,
               int64_t K, int G, int group_size, int64_t total_slots) {
  const int64_t slot = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (slot >= total_slots) return;
  const int lane = (int)(slot & 63);
  const int64_t tile = slot >> 6;
  const int64_t rb = tile / k_tiles, kb = tile - rb * k_tiles;
  const int r = lane & 15, q = lane >> 4;
  const UnpackConsts<BITS> kc_unpack;
  uint32_t w[BITS];
  load_tile_words<BITS>(packed + tile * tile_words(BITS), lane, w);
  _Float16* row = reinterpret_cast<_Float16*>(w_out) + (rb * 16 + r) * K + kb * 128 + q * 8;
  auto emit = [&](auto jtag) {
    constexpr int J = decltype(jtag)::value;
    uint32_t raw[4];
    raw_octet<BITS, J>(w, kc_unpack, raw);
    const int64_t k0 = kb * 128 + J * 32 + q * 8;
    const int64_t g = group_size == -1 ? 0 : k0 / group_size;
    const size_t so = ((size_t)rb * G + g) * 16 + r;
    const _Float16 s = reinterpret_cast<const _Float16*>(scales)[so];
    const _Float16 z = zeros ? reinterpret_cast<const _Float16*>(zeros)[so] : (_Float16)128.0f;
    H4 lo, hi;
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const int c = (int)code_from_raw<BITS>(raw, J, e) << (8 - BITS);
      const _Float16 diff = (_Float16)((float)c - (float)z);  // one fp16 rounding
      const _Float16 v = (_Float16)((float)s * (float)diff);  // and a second one
      if (e < 4) lo.h[e] = v; else hi.h[e - 4] = v;
    }
    *reinterpret_cast<uint4*>(row + J * 32) = make_uint4(lo.v.x, lo.v.y, hi.v.x, hi.v.y);
  };
  emit(std::integral_constant<int, 0>{});
  emit(std::integral_constant<int, 1>{});
  emit(std::integral_constant<int, 2>{});
  emit(std::integral_constant<int, 3>{});
}

// ---- master-resident bit planes (master_layout.h) --------------------------------------
// 32 codes of a lane slot from row-major uint8 [N, K]
__device__ __forceinline__ void read_lane_codes(const uint8_t* __restrict__ row, uint8_t (&c)[32]) {
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const uint2 v = *reinterpret_cast<const uint2*>(row + j * 32);
#pragma unroll
    for (int e = 0; e < 4; e++) {
      c[j * 8 + e] = (uint8_t)(v.x >> (8 * e));
      c[j * 8 + 4 + e] = (uint8_t)(v.y >> (8 * e));
    }
  }
}

// master codes [N, K] -> bit planes; one thread = one lane slot of one tile
__global__ void __launch_bounds__(256)
pack_master_kernel(const uint8_t* __restrict__ codes, uint32_t* __restrict__ out, int k_tiles,
                   int64_t K, int64_t total_slots) {
  const int64_t slot = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (slot >= total_slots) return;
  const int lane = (int)(slot & 63);
  const int64_t tile = slot >> 6;
  const int64_t rb = tile / k_tiles, kb = tile - rb * k_tiles;
  uint8_t c[32];
  read_lane_codes(codes + (rb * 16 + (lane & 15)) * K + kb * 128 + (lane >> 4) * 8, c);
  uint32_t w[8];
  master_encode_lane(c, w);
  uint32_t* t = out + tile * kMasterTileWords;
#pragma unroll
  for (int i = 0; i < 8; i++) t[master_word_offset(lane, i)] = w[i];
}

// bit planes -> codes sliced to BITS with the sequence the GEMM kernels run:
// SLICED_PACKED false: uint8 [N, K] (bit-exactness checks);
// SLICED_PACKED true : the pre-sliced tile layout of layout.h (input of the kernels that do not
//                      read the planes themselves)
template <int BITS, bool SLICED_PACKED>
__global__ void __launch_bounds__(256)
master_slice_kernel(const uint32_t* __restrict__ planes, void* __restrict__ out, int k_tiles,
                    int64_t K, int64_t total_slots) {
  const int64_t slot = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (slot >= total_slots) return;
  const int lane = (int)(slot & 63);
  const int64_t tile = slot >> 6;
  const int64_t rb = tile / k_tiles, kb = tile - rb * k_tiles;
  const uint32_t* t = planes + tile * kMasterTileWords;
  uint32_t w[8];
#pragma unroll
  for (int i = 0; i < 8; i++) w[i] = i < master_words(BITS) ? t[master_word_offset(lane, i)] : 0u;
  uint8_t c[32];
  master_decode_lane<BITS>(w, c);
  if constexpr (SLICED_PACKED) {
    uint32_t pw[BITS];
    Codec<BITS>::encode_lane(c, pw);
    uint32_t* o = static_cast<uint32_t*>(out) + tile * tile_words(BITS);
#pragma unroll
    for (int i = 0; i < BITS; i++) o[word_offset(BITS, lane, i)] = pw[i];
  } else {
    uint8_t* row = static_cast<uint8_t*>(out) + (rb * 16 + (lane & 15)) * K + kb * 128 + (lane >> 4) * 8;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      uint32_t lo = 0, hi = 0;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        lo |= (uint32_t)c[j * 8 + e] << (8 * e);
        hi |= (uint32_t)c[j * 8 + 4 + e] << (8 * e);
      }
      *reinterpret_cast<uint2*>(row + j * 32) = make_uint2(lo, hi);
    }
  }
}

inline unsigned blocks_for(int64_t n, int per_block) { return (unsigned)((n + per_block - 1) / per_block); }

}  // namespace

hipError_t launch_pack(const uint8_t* codes, int64_t N, int64_t K, int bits, int slice,
                       uint32_t* out, hipStream_t s) {
  const int k_tiles = (int)(K / 128);
  const int64_t slots = (N / 16) * (int64_t)k_tiles * 64;
  const dim3 grid(blocks_for(slots, 256)), block(256);
  switch (bits) {
    case 2: hipLaunchKernelGGL(pack_kernel<2>, grid, block, 0, s, codes, out, k_tiles, K, slots, slice); break;
    case 3: hipLaunchKernelGGL(pack_kernel<3>, grid, block, 0, s, codes, out, k_tiles, K, slots, slice); break;
    case 4: hipLaunchKernelGGL(pack_kernel<4>, grid, block, 0, s, codes, out, k_tiles, K, slots, slice); break;
    case 6: hipLaunchKernelGGL(pack_kernel<6>, grid, block, 0, s, codes, out, k_tiles, K, slots, slice); break;
    default: hipLaunchKernelGGL(pack_kernel<8>, grid, block, 0, s, codes, out, k_tiles, K, slots, slice); break;
  }
  return hipGetLastError();
}

hipError_t launch_unpack(const uint32_t* packed, int64_t N, int64_t K, int bits, uint8_t* codes,
                         hipStream_t s) {
  const int k_tiles = (int)(K / 128);
  const int64_t slots = (N / 16) * (int64_t)k_tiles * 64;
  const dim3 grid(blocks_for(slots, 256)), block(256);
  switch (bits) {
    case 2: hipLaunchKernelGGL(unpack_kernel<2>, grid, block, 0, s, packed, codes, k_tiles, K, slots); break;
    case 3: hipLaunchKernelGGL(unpack_kernel<3>, grid, block, 0, s, packed, codes, k_tiles, K, slots); break;
    case 4: hipLaunchKernelGGL(unpack_kernel<4>, grid, block, 0, s, packed, codes, k_tiles, K, slots); break;
    case 6: hipLaunchKernelGGL(unpack_kernel<6>, grid, block, 0, s, packed, codes, k_tiles, K, slots); break;
    default: hipLaunchKernelGGL(unpack_kernel<8>, grid, block, 0, s, packed, codes, k_tiles, K, slots); break;
  }
  return hipGetLastError();
}

hipError_t launch_pack_master(const uint8_t* codes, int64_t N, int64_t K, uint32_t* out, hipStream_t s) {
  const int k_tiles = (int)(K / 128);
  const int64_t slots = (N / 16) * (int64_t)k_tiles * 64;
  hipLaunchKernelGGL(pack_master_kernel, dim3(blocks_for(slots, 256)), dim3(256), 0, s, codes, out, k_tiles, K, slots);
  return hipGetLastError();
}

// sliced_packed: write the pre-sliced tile layout instead of uint8 [N, K]
hipError_t launch_master_slice(const uint32_t* planes, int64_t N, int64_t K, int bits, bool sliced_packed,
                               void* out, hipStream_t s) {
  const int k_tiles = (int)(K / 128);
  const int64_t slots = (N / 16) * (int64_t)k_tiles * 64;
  const dim3 grid(blocks_for(slots, 256)), block(256);
#define MATGPTQ_MS(B)                                                                                         \
  case B:                                                                                                     \
    if (sliced_packed) hipLaunchKernelGGL((master_slice_kernel<B, true>), grid, block, 0, s, planes, out, k_tiles, K, slots); \
    else hipLaunchKernelGGL((master_slice_kernel<B, false>), grid, block, 0, s, planes, out, k_tiles, K, slots);  \
    break;
  switch (bits) {
    MATGPTQ_MS(2)
    MATGPTQ_MS(3)
    MATGPTQ_MS(4)
    MATGPTQ_MS(6)
    default:
      if (sliced_packed) hipLaunchKernelGGL((master_slice_kernel<8, true>), grid, block, 0, s, planes, out, k_tiles, K, slots);
      else hipLaunchKernelGGL((master_slice_kernel<8, false>), grid, block, 0, s, planes, out, k_tiles, K, slots);
      break;
  }
#undef MATGPTQ_MS
  return hipGetLastError();
}

hipError_t launch_slice(const uint8_t* in, int64_t count, int bits, uint8_t* out, hipStream_t s) {
  const dim3 grid(blocks_for((count + 3) / 4, 256)), block(256);
  hipLaunchKernelGGL(slice_kernel, grid, block, 0, s, in, out, count, bits);
  return hipGetLastError();
}

hipError_t launch_reorder(const uint16_t* in, int64_t N, int64_t G, uint16_t* out, hipStream_t s) {
  const int64_t total = N * G;
  const dim3 grid(blocks_for(total, 256)), block(256);
  hipLaunchKernelGGL(reorder_kernel, grid, block, 0, s, in, out, G, total);
  return hipGetLastError();
}

hipError_t launch_dequant(int bits, int group_size, int64_t N, int64_t K, const uint32_t* packed,
                          const uint16_t* scales, const uint16_t* zeros, uint16_t* w,
                          hipStream_t s) {
  const int k_tiles = (int)(K / 128);
  const int G = group_size == -1 ? 1 : (int)(K / group_size);
  const int64_t slots = (N / 16) * (int64_t)k_tiles * 64;
  const dim3 grid(blocks_for(slots, 256)), block(256);
#define MATGPTQ_DQ(B) hipLaunchKernelGGL(dequant_kernel<B>, grid, block, 0, s, packed, scales, zeros, w, k_tiles, K, G, group_size, slots)
  switch (bits) {
    case 2: MATGPTQ_DQ(2); break;
    case 3: MATGPTQ_DQ(3); break;
    case 4: MATGPTQ_DQ(4); break;
    case 6: MATGPTQ_DQ(6); break;
    default: MATGPTQ_DQ(8); break;
  }
#undef MATGPTQ_DQ
  return hipGetLastError();
}

}  // namespace matgptq
