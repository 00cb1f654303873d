// Mid-batch kernel (a few batch rows up to a few hundred): the K dimension is split inside the
// workgroup.
// Compiled once per bitwidth with -DMATGPTQ_BITS=b.
//
// At these batch sizes a layer has few output tiles: a kernel that gives every workgroup a
// tile of outputs and walks K serially leaves most of the GPU idle and is bound by the latency
// of one K walk (the reference's tensor-core kernel has this shape, one 16 x 8 tile per block,
// inference_lib/matgptq_cuda/csrc/matgptq_gemm.cu:337-634).  Here
//
//  * a workgroup of eight waves owns R row blocks of 16 weight rows and 16*MB activation rows;
//    wave w takes the K tiles w, w + 8, ... of those rows, so a layer with N / (16 R) x M / (16 MB)
//    output tiles still runs eight times as many waves, each with a short K walk;
//  * each wave dequantises its tiles from registers into the 16x32 MFMA operand (the same
//    arithmetic as the large-batch kernel: fp16 weights times fp16 activations, or bf16 weights,
//    formed in fp32 and rounded once, times the bf16 activations as stored).  No two waves of a workgroup read the same
//    activations, so every wave stages its own: buffer_load ... lds copies the 16*MB x 128
//    activations of a tile from global memory straight into the wave's private LDS buffer,
//    256 contiguous bytes per 16 lanes (an operand read straight from global memory
//    would touch sixteen rows with sixteen adjacent lanes).  16-byte chunk c of row r lies at
//    position c ^ (r & 15) of the LDS row, so the sixteen lanes of an operand read hit sixteen
//    different bank groups;
//  * a wave has one LDS buffer and two register sets of codes, scales and zeros.  At the start
//    of a tile it waits for its own copies and loads (vmcnt(0): nothing younger is in flight),
//    reads the tile's operands from LDS into registers, and only then requests the next tile
//    into the same buffer and the other register set, which arrive while this tile is
//    dequantised and multiplied.  One buffer instead of two keeps the LDS of a workgroup at
//    32 KB per 16 batch rows, so that several workgroups share a CU: a walk is short (K / 1024
//    tiles) and what hides the memory latency is the number of waves, not the depth of a
//    ring (a four-deep ring at 128 KB per workgroup measured 10-30 % slower).  There is no
//    barrier in the loop;
//  * every load is branch-free (tiles beyond K, rows beyond M or N go through a zero-length
//    buffer descriptor or an out-of-range offset);
//  * the eight partial sums meet in LDS once, at the end; the threads add them and store four
//    consecutive output columns each.
//
// The activations are re-read once per workgroup column (N / (16 R) times in total, from L2):
// that traffic, not the weights, bounds this kernel, which is why R grows with N.
#include "tile_format.h"

#ifndef MATGPTQ_BITS
#error "compile with -DMATGPTQ_BITS={2,3,4,6,8}"
#endif

namespace matgptq {

namespace {

constexpr int kBits = MATGPTQ_BITS;
constexpr int kWaves = 8;

// Stages of a wave's ring: as many as fit 128 KB of LDS per workgroup.
// LDS of a workgroup: per wave one activation buffer of 16*MB rows x 256 bytes; the partial
// sums (16 bytes per lane, row block and batch block per wave) reuse them after the loop.
constexpr int skinny_lds_bytes(int r, int mb) {
  const int stage = kWaves * mb * 16 * 256, sums = kWaves * r * mb * 64 * 16;
  return stage > sums ? stage : sums;
}

// MASTER: `a.packed` holds the master-resident bit planes (master_layout.h); the slice to BITS,
// rounding and saturation happen in registers on the way to the raw fp16 pairs.
template <int BITS, int GROUP, bool ZP, int R, int MB, bool MASTER>
__global__ void __launch_bounds__(64 * kWaves, 2)
skinny_kernel(const GemmArgs a, int n_tiles, int m_tiles) {
  using Fmt = TileFormat<BITS, MASTER>;
  constexpr int GPT = GROUP == 32 ? 4 : 1;
  constexpr int kStage = MB * 16 * 256;  // bytes of one activation buffer
  constexpr int NS = 2;  // register sets of codes, scales, zeros
  __shared__ __align__(16) unsigned char smem[skinny_lds_bytes(R, MB)];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15;
  const int q = lane >> 4;

  // Workgroup ids go round-robin over the 8 XCDs: remapped so that the workgroups of one XCD
  // walk consecutive activation tiles of the same weight rows and share those rows in its L2.
  const int total = n_tiles * m_tiles;
  int lid = blockIdx.x;
  if ((total & 7) == 0) lid = (blockIdx.x & 7) * (total >> 3) + (blockIdx.x >> 3);
  const int nt = lid / m_tiles;
  const int m0 = (lid - nt * m_tiles) * (16 * MB);
  const int rb_first = nt * R;

  constexpr uint32_t tile_bytes = Fmt::kTileBytes;
  const uint32_t rb_bytes = (uint32_t)a.k_tiles * tile_bytes;
  const uint32_t w_bytes = (uint32_t)a.row_blocks * rb_bytes;
  const uint32_t aux_bytes = (uint32_t)a.row_blocks * a.G * 32;  // scales / zeros: [N/16][G][16] halves
  const uint32_t x_bytes = (uint32_t)a.M * (uint32_t)a.K * 2u;

  float4v acc[R][MB];
#pragma unroll
  for (int rr = 0; rr < R; rr++)
#pragma unroll
    for (int i = 0; i < MB; i++) acc[rr][i] = float4v{0.f, 0.f, 0.f, 0.f};

  const typename Fmt::Consts kc_unpack;
  const float kc_zero = __uint_as_float(opaque_vgpr(0u));  // a zero the optimiser cannot see through
  // codes, scales and zeros of the tile in use and of the next one; scales and zeros stay as
  // loaded and are converted where they are used
  uint32_t wr[NS][R][Fmt::kWords], sr[NS][R][GPT], zr[NS][R][GPT];

  auto load_weights = [&](uint32_t (&w)[R][Fmt::kWords], uint32_t (&s)[R][GPT], uint32_t (&z)[R][GPT], int kb) {
#pragma unroll
    for (int rr = 0; rr < R; rr++) {
      const int rb = rb_first + rr;
      const bool valid = rb < a.row_blocks && kb < a.k_tiles;
      const BufRsrc wr = make_rsrc(a.packed, valid ? w_bytes : 0u);
      const BufRsrc sr = make_rsrc(a.scales, valid ? aux_bytes : 0u);
      const BufRsrc zr = make_rsrc(ZP ? a.zeros : a.scales, valid ? aux_bytes : 0u);
      Fmt::template load<0>(wr, (uint32_t)rb * rb_bytes + (uint32_t)kb * tile_bytes, lane, w[rr]);
#pragma unroll
      for (int gg = 0; gg < GPT; gg++) {
        const uint32_t g = GROUP == -1 ? 0u : (uint32_t)kb * GPT + gg;
        const uint32_t so = ((uint32_t)rb * a.G + g) * 32;  // bytes
        s[rr][gg] = __builtin_amdgcn_raw_buffer_load_b16(sr, r16 * 2, so, 0);
        if constexpr (ZP) z[rr][gg] = __builtin_amdgcn_raw_buffer_load_b16(zr, r16 * 2, so, 0);
        else z[rr][gg] = 0u;
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  // Copy of one tile's activations: instruction i moves rows 4i .. 4i+3 (lane l: row 4i + l/16,
  // LDS position l%16, which holds chunk (l%16) ^ (row & 15) of the row's 256 bytes).
  unsigned char* const stage = smem + wave * kStage;
  uint32_t dma_voff[4 * MB];
#pragma unroll
  for (int i = 0; i < 4 * MB; i++) {
    const int row = 4 * i + (lane >> 4);
    const int c = (lane & 15) ^ (row & 15);
    const uint32_t m = (uint32_t)(m0 + row);
    dma_voff[i] = m < (uint32_t)a.M ? m * (uint32_t)a.K * 2u + c * 16 : x_bytes;
  }
  auto dma = [&](int kb) {
    const BufRsrc xres = make_rsrc(a.x, kb < a.k_tiles ? x_bytes : 0u);
#pragma unroll
    for (int i = 0; i < 4 * MB; i++)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          xres, (__attribute__((address_space(3))) void*)(stage + i * 1024), 16, (int)dma_voff[i],
          (int)((uint32_t)kb * 256u), 0, 0);  // (int: the builtin's own parameter type)
    __builtin_amdgcn_sched_barrier(0);
  };
  // operand of batch rows i*16 + r16, columns [j*32 + q*8, +8) of the tile: chunk 4j + q
  auto read_frag = [&](int i, int j) {
    return *reinterpret_cast<const half8*>(stage + (i * 16 + r16) * 256 + (((4 * j + q) ^ r16) * 16));
  };

  auto dequant_step = [&](Frag (&aw)[R], const uint32_t (&w)[R][Fmt::kWords], const uint32_t (&s)[R][GPT],
                          const uint32_t (&z)[R][GPT], auto jtag) {
    constexpr int J = decltype(jtag)::value;
#pragma unroll
    for (int rr = 0; rr < R; rr++) {
      const int gg = GROUP == 32 ? J : 0;
      if constexpr (kBf16) {
        // bf16 storage: the activations go to the bf16 matrix instruction as stored; the weights
        // are formed in fp32 from scale * 2^(8-b) and scale * (zero - 128) and rounded to bf16 once
        const float s0 = bf16_bits_to_float(s[rr][gg]);
        const float sm = s0 * (float)(1 << (8 - BITS));
        float sz = kc_zero;
        if constexpr (ZP) sz = s0 * (bf16_bits_to_float(z[rr][gg]) - 128.0f);
        dequant_octet_bf16_fmt<Fmt, BITS, J>(w[rr], kc_unpack, sm, sz, aw[rr]);
      } else {
        // fp16 storage: scale * 2^(8-b) and scale * (zero - 128)
        const _Float16 s0 = __builtin_bit_cast(_Float16, (uint16_t)s[rr][gg]);
        const _Float16 s1 = (_Float16)((float)s0 * (float)(1 << (8 - BITS)));  // scale * m
        _Float16 z1 = (_Float16)0.f;
        if constexpr (ZP) z1 = s0 * (__builtin_bit_cast(_Float16, (uint16_t)z[rr][gg]) - (_Float16)128.0f);
        const half2v sc = {s1, s1};
        const half2v zr = {z1, z1};
        dequant_octet_fmt<Fmt, BITS, J, ZP>(w[rr], kc_unpack, zr, sc, aw[rr]);
      }
    }
  };

  // Tile t of the walk (K tile kb = wave + 8 t), codes in register set `btag`.
  auto tile = [&](int t, auto btag) {
    constexpr int B = decltype(btag)::value;
    const int kb = wave + t * kWaves;
    // everything this wave has requested has arrived: the copy of this tile's activations and
    // this tile's codes were the last requests
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (0 << 8) | (0 << 14));  // vmcnt(0), lgkmcnt(0)
    __builtin_amdgcn_sched_barrier(0);
    half8 xf[4][MB];
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int i = 0; i < MB; i++) xf[j][i] = read_frag(i, j);
    // the buffer is free once these reads have returned: request the next tile
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(15 | (7 << 4) | (0 << 8) | (3 << 14));  // lgkmcnt(0)
    __builtin_amdgcn_sched_barrier(0);
    dma(kb + kWaves);
    load_weights(wr[B ^ 1], sr[B ^ 1], zr[B ^ 1], kb + kWaves);
    if (kb < a.k_tiles) {
      auto one = [&](auto jtag) {
        constexpr int J = decltype(jtag)::value;
        Frag aw[R];
        dequant_step(aw, wr[B], sr[B], zr[B], jtag);
#pragma unroll
        for (int i = 0; i < MB; i++) {
#pragma unroll
          for (int rr = 0; rr < R; rr++) {
            if constexpr (kBf16)
              acc[rr][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, aw[rr].h),
                                                                  __builtin_bit_cast(bf16x8, xf[J][i]), acc[rr][i], 0, 0, 0);
            else
              acc[rr][i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aw[rr].h, xf[J][i], acc[rr][i], 0, 0, 0);
          }
        }
      };
      one(std::integral_constant<int, 0>{});
      one(std::integral_constant<int, 1>{});
      one(std::integral_constant<int, 2>{});
      one(std::integral_constant<int, 3>{});
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  const int walk = (a.k_tiles + kWaves - 1) / kWaves;  // tiles of the longest walk
  __builtin_amdgcn_sched_barrier(0);
  dma(wave);
  load_weights(wr[0], sr[0], zr[0], wave);
  for (int t = 0; t < walk; t += 2) {
    tile(t, std::integral_constant<int, 0>{});
    tile(t + 1, std::integral_constant<int, 1>{});
  }

  // The eight partial sums of every output meet in LDS (over the activation buffers: every
  // wave has to be done with its own first); thread t adds the eight float4 of one (row
  // block, batch block, lane) and stores rows (weight rows) 4q..4q+3 of column (batch row) r16.
  __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (0 << 8) | (0 << 14));  // nothing in flight into LDS any more
  __syncthreads();
  float4v* const red = reinterpret_cast<float4v*>(smem);
#pragma unroll
  for (int rr = 0; rr < R; rr++)
#pragma unroll
    for (int i = 0; i < MB; i++) red[((wave * R + rr) * MB + i) * 64 + lane] = acc[rr][i];
  __syncthreads();
  // (R * MB * 64 outputs of four values each: up to twice the threads of the workgroup)
  for (int ot = tid; ot < R * MB * 64; ot += 64 * kWaves) {
    float4v sum = red[ot];
#pragma unroll
    for (int w = 1; w < kWaves; w++) sum += red[w * R * MB * 64 + ot];
    const int l = ot & 63, ri = ot >> 6;
    const int rb = rb_first + ri / MB;
    const int m = m0 + (ri % MB) * 16 + (l & 15);
    if (rb < a.row_blocks && m < a.M) {
      uint16_t o[4];
#pragma unroll
      for (int e = 0; e < 4; e++) o[e] = float_to_storage(sum[e]);
      *reinterpret_cast<uint2*>(a.y + (size_t)m * a.N + (size_t)rb * 16 + 4 * (l >> 4)) =
          make_uint2((uint32_t)o[0] | ((uint32_t)o[1] << 16), (uint32_t)o[2] | ((uint32_t)o[3] << 16));
    }
  }
}

template <int GROUP, bool ZP, int R, int MB, bool MASTER>
hipError_t launch_r(const GemmArgs& a, hipStream_t stream) {
  const int n_tiles = (a.row_blocks + R - 1) / R;
  const int m_tiles = (a.M + 16 * MB - 1) / (16 * MB);
  const dim3 grid(n_tiles * m_tiles), block(64 * kWaves);
  hipLaunchKernelGGL((skinny_kernel<kBits, GROUP, ZP, R, MB, MASTER>), grid, block, 0, stream, a, n_tiles, m_tiles);
  return hipGetLastError();
}

template <int GROUP, bool ZP, int MB, bool MASTER>
hipError_t launch_rows(const GemmArgs& a, int r, hipStream_t s) {
  // (four row blocks fit the register budget of two waves per SIMD up to 6 bits and with one
  // scale and zero per tile and row block; group 32 carries four; the master planes are eight
  // words per lane from 6 bits on)
  // (eight row blocks: pre-sliced codes up to 4 bits, 32 batch rows)
  if constexpr (GROUP != 32 && kBits <= 4 && !MASTER && MB == 2) {
    if (r >= 8) return launch_r<GROUP, ZP, 8, MB, MASTER>(a, s);
  }
  if constexpr (GROUP != 32 && kBits <= (MASTER ? 4 : 6)) {
    if (r >= 4) return launch_r<GROUP, ZP, 4, MB, MASTER>(a, s);
  }
  if (r >= 2) return launch_r<GROUP, ZP, 2, MB, MASTER>(a, s);
  return launch_r<GROUP, ZP, 1, MB, MASTER>(a, s);
}

template <int GROUP, bool ZP, bool MASTER>
hipError_t launch_batch(const GemmArgs& a, int r, int mb, hipStream_t s) {
  if (mb >= 4) return launch_rows<GROUP, ZP, 4, MASTER>(a, r, s);
  return mb >= 2 ? launch_rows<GROUP, ZP, 2, MASTER>(a, r, s) : launch_rows<GROUP, ZP, 1, MASTER>(a, r, s);
}

template <int GROUP, bool ZP>
hipError_t launch_storage(const GemmArgs& a, int r, int mb, bool master, hipStream_t s) {
  return master ? launch_batch<GROUP, ZP, true>(a, r, mb, s) : launch_batch<GROUP, ZP, false>(a, r, mb, s);
}

}  // namespace

#define MATGPTQ_CAT2(a, b) a##b
#define MATGPTQ_CAT(a, b) MATGPTQ_CAT2(a, b)
// r: row blocks of 16 weight rows per workgroup (1, 2, 4 or 8); mb: blocks of 16 batch rows (1, 2 or 4)
#if MATGPTQ_BF16
#define MATGPTQ_LAUNCH_NAME MATGPTQ_CAT(MATGPTQ_CAT(launch_skinny_b, MATGPTQ_BITS), _bf16)
#else
#define MATGPTQ_LAUNCH_NAME MATGPTQ_CAT(launch_skinny_b, MATGPTQ_BITS)
#endif
// master: `a.packed` holds master-resident bit planes
hipError_t MATGPTQ_LAUNCH_NAME(const GemmArgs& a, int group_size, int r, int mb, bool master, hipStream_t stream) {
  const bool zp = a.zeros != nullptr;
  if (group_size == 128)
    return zp ? launch_storage<128, true>(a, r, mb, master, stream) : launch_storage<128, false>(a, r, mb, master, stream);
  if (group_size == 32)
    return zp ? launch_storage<32, true>(a, r, mb, master, stream) : launch_storage<32, false>(a, r, mb, master, stream);
  return zp ? launch_storage<-1, true>(a, r, mb, master, stream) : launch_storage<-1, false>(a, r, mb, master, stream);
}

}  // namespace matgptq
