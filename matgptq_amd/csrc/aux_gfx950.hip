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

// ---- the tail of K = 128 t + 64 (layout.h): 64 columns per row as a bitstream ---------------
// one thread = one row
__global__ void __launch_bounds__(256)
pack_tail_kernel(const uint8_t* __restrict__ codes, uint32_t* __restrict__ tail, int64_t N, int64_t K,
                 int bits, int slice) {
  const int64_t n = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= N) return;
  const uint8_t* src = codes + n * K + (K - kTailCols);
  uint8_t c[kTailCols];
  for (int k = 0; k < kTailCols; k++) c[k] = slice ? slice_code(src[k], bits) : src[k];
  uint32_t row[16];
  tail_encode_row(c, bits, row);
  for (int i = 0; i < tail_row_words(bits); i++) tail[n * tail_row_words(bits) + i] = row[i];
}

// one thread = one code
__global__ void __launch_bounds__(256)
unpack_tail_kernel(const uint32_t* __restrict__ tail, uint8_t* __restrict__ codes, int64_t N, int64_t K, int bits) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= N * kTailCols) return;
  const int64_t n = i / kTailCols;
  const int k = (int)(i - n * kTailCols);
  codes[n * K + (K - kTailCols) + k] = (uint8_t)tail_code(tail + n * tail_row_words(bits), bits, k);
}

// scale and zero of (row n, column k) from the reordered [N/16][G][16] tensors, as float
template <bool BF16>
__device__ __forceinline__ void tail_scale_zero(const uint16_t* scales, const uint16_t* zeros, int64_t n, int64_t k,
                                                int G, int group_size, float& s, float& z) {
  const int64_t g = group_size == -1 ? 0 : k / group_size;
  const size_t so = ((size_t)(n >> 4) * G + g) * 16 + (n & 15);
  if constexpr (BF16) {
    s = bf16_bits_to_float(scales[so]);
    z = zeros ? bf16_bits_to_float(zeros[so]) : 128.0f;
  } else {
    s = (float)__builtin_bit_cast(_Float16, scales[so]);
    z = zeros ? (float)__builtin_bit_cast(_Float16, zeros[so]) : 128.0f;
  }
}

// one weight the way dequantize() forms it on tensors of the storage type: the difference and the
// product are each rounded to that type
template <bool BF16>
__device__ __forceinline__ float tail_weight(uint32_t code, int bits, float s, float z) {
  const float d = (float)(int)(code << (8 - bits)) - z;
  if constexpr (BF16) {
    const float dr = bf16_bits_to_float(float_to_bf16_bits(d));
    return bf16_bits_to_float(float_to_bf16_bits(s * dr));
  } else {
    const float dr = (float)(_Float16)d;
    return (float)(_Float16)(s * dr);
  }
}

// dense dequantise, tail columns: one thread = one weight (fp16 storage, like dequant_kernel)
__global__ void __launch_bounds__(256)
dequant_tail_kernel(const uint32_t* __restrict__ tail, const uint16_t* __restrict__ scales,
                    const uint16_t* __restrict__ zeros, uint16_t* __restrict__ w_out, int64_t N, int64_t K,
                    int G, int group_size, int bits) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= N * kTailCols) return;
  const int64_t n = i / kTailCols;
  const int64_t k = (K - kTailCols) + (i - n * kTailCols);
  float s, z;
  tail_scale_zero<false>(scales, zeros, n, k, G, group_size, s, z);
  const float w = tail_weight<false>(tail_code(tail + n * tail_row_words(bits), bits, (int)(i - n * kTailCols)), bits, s, z);
  w_out[n * K + k] = __builtin_bit_cast(uint16_t, (_Float16)w);
}

// Y[m][n] += sum over the tail columns of X[m][k] W[n][k]: runs after the GEMM over the tiles has
// written Y.  A workgroup = 16 weight rows x 16 lanes of batch rows; a thread keeps the 64 weights
// of its row in registers and walks `m_per_block` / 16 batch rows.  N x 64 weights against a GEMM of
// N x 128 t: a plain vector-ALU kernel is enough.
template <bool BF16>
__global__ void __launch_bounds__(256)
tail_gemm_kernel(const uint32_t* __restrict__ tail, const uint16_t* __restrict__ scales,
                 const uint16_t* __restrict__ zeros, const uint16_t* __restrict__ x, uint16_t* __restrict__ y,
                 int N, int K, int M, int G, int group_size, int bits, int m_per_block) {
  const int n = blockIdx.x * 16 + (threadIdx.x & 15);
  const int ml = threadIdx.x >> 4;
  const int K0 = K - kTailCols;
  const uint32_t* row = tail + (size_t)n * tail_row_words(bits);
  float w[kTailCols];
#pragma unroll
  for (int k8 = 0; k8 < kTailCols / 32; k8++) {  // a scale per 32 columns at most
    float s, z;
    tail_scale_zero<BF16>(scales, zeros, n, K0 + k8 * 32, G, group_size, s, z);
#pragma unroll
    for (int k = 0; k < 32; k++) w[k8 * 32 + k] = tail_weight<BF16>(tail_code(row, bits, k8 * 32 + k), bits, s, z);
  }
  const int m_end = min(M, (int)(blockIdx.y + 1) * m_per_block);
  for (int m = blockIdx.y * m_per_block + ml; m < m_end; m += 16) {
    const uint4* xp = reinterpret_cast<const uint4*>(x + (size_t)m * K + K0);
    float acc = 0.f;
#pragma unroll
    for (int c = 0; c < kTailCols / 8; c++) {
      const uint4 v = xp[c];
      const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int e = 0; e < 4; e++) {
        float lo, hi;
        if constexpr (BF16) {
          lo = bf16_bits_to_float(u[e] & 0xffffu);
          hi = bf16_bits_to_float(u[e] >> 16);
        } else {
          lo = (float)__builtin_bit_cast(_Float16, (uint16_t)(u[e] & 0xffffu));
          hi = (float)__builtin_bit_cast(_Float16, (uint16_t)(u[e] >> 16));
        }
        acc = __builtin_fmaf(lo, w[c * 8 + 2 * e], acc);
        acc = __builtin_fmaf(hi, w[c * 8 + 2 * e + 1], acc);
      }
    }
    uint16_t* yp = y + (size_t)m * N + n;
    if constexpr (BF16) *yp = (uint16_t)float_to_bf16_bits(bf16_bits_to_float(*yp) + acc);
    else *yp = __builtin_bit_cast(uint16_t, (_Float16)((float)__builtin_bit_cast(_Float16, *yp) + acc));
  }
}

// Reads `chunks` 16-byte chunks once and keeps nothing: wave w of a workgroup of eight requests
// four consecutive KiB at once, like a wave of the batch-1 GEMM kernel does with its four tiles.
__global__ void __launch_bounds__(512)
read_probe_kernel(const u32x4* __restrict__ p, size_t chunks, uint32_t* __restrict__ sink) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const size_t base = ((size_t)blockIdx.x * 8 + wave) * 256 + lane;
  u32x4 v[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const size_t c = base + (size_t)i * 64;
    v[i] = c < chunks ? __builtin_nontemporal_load(p + c) : u32x4{0u, 0u, 0u, 0u};
  }
  uint32_t acc = 0;
#pragma unroll
  for (int i = 0; i < 4; i++) acc ^= v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
  if (acc == 0x9e3779b9u && sink) sink[0] = acc;  // (keeps the loads alive; `sink` is null)
}

inline unsigned blocks_for(int64_t n, int per_block) { return (unsigned)((n + per_block - 1) / per_block); }

// first word of the tail: behind the tiles of all row blocks
inline int64_t tail_offset_words(int64_t N, int64_t K, int bits) { return (N / 16) * (K / 128) * tile_words(bits); }

}  // namespace

hipError_t launch_read_probe(const void* buf, size_t bytes, hipStream_t s) {
  const size_t chunks = bytes / 16;
  hipLaunchKernelGGL(read_probe_kernel, dim3(blocks_for((int64_t)chunks, 2048)), dim3(512), 0, s,
                     static_cast<const u32x4*>(buf), chunks, static_cast<uint32_t*>(nullptr));
  return hipGetLastError();
}

// Adds the product over the last 64 columns (K = 128 t + 64) to Y; `a` as for the GEMM kernels.
hipError_t launch_tail_gemm(int bits, bool bf16, const GemmArgs& a, int group_size, hipStream_t s) {
  const uint32_t* tail = a.packed + tail_offset_words(a.N, a.K, bits);
  const int m_per_block = 128;
  const dim3 grid(a.N / 16, (a.M + m_per_block - 1) / m_per_block), block(256);
  if (bf16)
    hipLaunchKernelGGL(tail_gemm_kernel<true>, grid, block, 0, s, tail, a.scales, a.zeros, a.x, a.y, a.N, a.K, a.M, a.G,
                       group_size, bits, m_per_block);
  else
    hipLaunchKernelGGL(tail_gemm_kernel<false>, grid, block, 0, s, tail, a.scales, a.zeros, a.x, a.y, a.N, a.K, a.M, a.G,
                       group_size, bits, m_per_block);
  return hipGetLastError();
}

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
  if (K % 128 != 0)
    hipLaunchKernelGGL(pack_tail_kernel, dim3(blocks_for(N, 256)), block, 0, s, codes, out + tail_offset_words(N, K, bits),
                       N, K, bits, slice);
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
  if (K % 128 != 0)
    hipLaunchKernelGGL(unpack_tail_kernel, dim3(blocks_for(N * kTailCols, 256)), block, 0, s,
                       packed + tail_offset_words(N, K, bits), codes, N, K, bits);
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
  if (K % 128 != 0)
    hipLaunchKernelGGL(dequant_tail_kernel, dim3(blocks_for(N * kTailCols, 256)), block, 0, s,
                       packed + tail_offset_words(N, K, bits), scales, zeros, w, N, K, G, group_size, bits);
  return hipGetLastError();
}

}  // namespace matgptq
