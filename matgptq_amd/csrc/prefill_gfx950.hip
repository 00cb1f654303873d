// Prefill-regime kernel (M > 16): dense contraction on the matrix cores.
// Compiled once per bitwidth with -DMATGPTQ_BITS=b.  The reference has no kernel
// of this kind: its tensor-core path re-reads and re-dequantises every weight
// once per eight batch rows (inference_lib/matgptq_cuda/csrc/matgptq_gemm.cu:337-634,961-963).
//
//  * a workgroup of four waves owns TM = 16*MT activation rows and 64*RBW weight
//    rows; wave w owns the RBW row blocks [w*RBW, +RBW) of that range, so every
//    packed code is dequantised by exactly one wave, straight from registers into
//    the 16x32 MFMA operand, as  fp16(scale * fp16((c << (8-b)) - zero)),  the value
//    the reference's dequantize() gives the weight;
//  * the activation tile is staged through LDS (double buffered, 64 columns per
//    stage, rows padded by 16 bytes so that the 16-byte operand reads of 16 rows
//    fall into distinct banks) and shared by the four waves;
//  * fp32 accumulators live in registers for the whole K loop; the epilogue packs
//    four consecutive output columns per lane into one 8-byte store.
//
// Workgroup ids are remapped so that the workgroups of one XCD (ids congruent
// modulo 8) walk consecutive activation tiles of the same weight rows and share
// those rows in their L2.
#include "device_common.h"

#ifndef MATGPTQ_BITS
#error "compile with -DMATGPTQ_BITS={2,3,4,6,8}"
#endif

namespace matgptq {

namespace {

constexpr int kBits = MATGPTQ_BITS;
constexpr int kXs = 64;          // activation columns per LDS stage
constexpr int kXsPitch = kXs + 8;  // halves per LDS row

// One raw pair -> two weights.  u = c - 2^(b-1) is exact; with a zero point
// v = m*u - (zero - 128) = (c << (8-b)) - zero is rounded once (exact for integral
// zeros) and multiplied by the scale; without, `scale` already carries the factor
// m = 2^(8-b) (a power of two, so the single rounding of the product is unchanged).
template <int BITS, int P, bool ZP>
__device__ __forceinline__ half2v dequant_pair(uint32_t raw, half2v zrel, half2v scale) {
  const half2v u = centre_raw<P>(raw, Codec<BITS>::kCentre);
  if constexpr (ZP) {
    constexpr float m = (float)(1 << (8 - BITS));
    const half2v v = __builtin_elementwise_fma(u, h2_splat(m), -zrel);
    return v * scale;
  } else {
    return u * scale;
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

// two waves per SIMD whenever the accumulators leave room for it
constexpr int prefill_min_waves(int rbw, int mt) { return rbw * mt * 4 <= 128 ? 2 : 1; }

template <int BITS, int GROUP, bool ZP, int RBW, int MT>
__global__ void __launch_bounds__(256, prefill_min_waves(RBW, MT))
prefill_kernel(const GemmArgs a, int n_tiles, int m_tiles) {
  constexpr int TM = 16 * MT;
  constexpr int GPT = GROUP == 32 ? 4 : 1;
  constexpr int XCHUNKS = TM * (kXs / 8) / 256;  // 16-byte chunks per thread per stage
  static_assert(TM * (kXs / 8) % 256 == 0, "activation tile must split evenly over 256 threads");
  __shared__ __align__(16) _Float16 xs[2][TM * kXsPitch];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: tile offsets stay scalar
  const int r16 = lane & 15;
  const int q = lane >> 4;

  // XCD-aware tile order
  const int total = n_tiles * m_tiles;
  int lid = blockIdx.x;
  if ((total & 7) == 0) lid = (blockIdx.x & 7) * (total >> 3) + (blockIdx.x >> 3);
  const int nt = lid / m_tiles;
  const int mtile = lid - nt * m_tiles;
  const int m0 = mtile * TM;
  const int rb_first = (nt * 4 + wave) * RBW;

  constexpr uint32_t tile_bytes = (uint32_t)tile_words(BITS) * 4;
  const uint32_t rb_bytes = (uint32_t)a.k_tiles * tile_bytes;
  const BufRsrc wres = make_rsrc(a.packed, (uint32_t)a.row_blocks * rb_bytes);
  const uint32_t aux_bytes = (uint32_t)a.row_blocks * a.G * 32;  // scales / zeros: [N/16][G][16] halves
  const BufRsrc sres = make_rsrc(a.scales, aux_bytes);
  const BufRsrc zres = make_rsrc(ZP ? a.zeros : a.scales, aux_bytes);

  float4v acc[RBW][MT];
#pragma unroll
  for (int rr = 0; rr < RBW; rr++)
#pragma unroll
    for (int mt = 0; mt < MT; mt++) acc[rr][mt] = float4v{0.f, 0.f, 0.f, 0.f};

  const UnpackConsts<BITS> kc_unpack;
  uint32_t wcur[RBW][BITS], wnxt[RBW][BITS];
  _Float16 scur[RBW][GPT], snxt[RBW][GPT];
  _Float16 zcur[RBW][GPT], znxt[RBW][GPT];

  auto load_weights = [&](uint32_t (&w)[RBW][BITS], _Float16 (&s)[RBW][GPT], _Float16 (&z)[RBW][GPT],
                          int kb) {
#pragma unroll
    for (int rr = 0; rr < RBW; rr++) {
      const int rb = rb_first + rr;
#ifdef MATGPTQ_DEBUG_NOWLOAD
      if (rb < a.row_blocks && kb == 0) {
#else
      if (rb < a.row_blocks) {
#endif
        load_tile_words<BITS, 0>(wres, (uint32_t)rb * rb_bytes + (uint32_t)kb * tile_bytes, lane, w[rr]);
#pragma unroll
        for (int gg = 0; gg < GPT; gg++) {
          const uint32_t g = GROUP == -1 ? 0u : (uint32_t)kb * GPT + gg;
          const uint32_t so = ((uint32_t)rb * a.G + g) * 32;  // bytes
          s[rr][gg] = __builtin_bit_cast(_Float16, (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(sres, r16 * 2, so, 0));
          if constexpr (ZP)
            z[rr][gg] = __builtin_bit_cast(_Float16, (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(zres, r16 * 2, so, 0)) -
                        (_Float16)128.0f;
        }
      } else {
#pragma unroll
        for (int i = 0; i < BITS; i++) w[rr][i] = 0;
#pragma unroll
        for (int gg = 0; gg < GPT; gg++) { s[rr][gg] = (_Float16)0.0f; z[rr][gg] = (_Float16)0.0f; }
      }
    }
  };

  uint4 xreg[XCHUNKS];
  auto load_x = [&](int h) {  // columns [h*64, +64)
#pragma unroll
    for (int c = 0; c < XCHUNKS; c++) {
      const int chunk = tid + c * 256;
      const int row = chunk >> 3, col8 = chunk & 7;
      const int m = m0 + row;
      xreg[c] = make_uint4(0u, 0u, 0u, 0u);
#ifdef MATGPTQ_DEBUG_NOXLOAD
      if (m < -1)
#else
      if (m < a.M)
#endif
        xreg[c] = *reinterpret_cast<const uint4*>(a.x + (size_t)m * a.K + (size_t)h * kXs + col8 * 8);
    }
  };
  auto store_x = [&](int buf) {
#pragma unroll
    for (int c = 0; c < XCHUNKS; c++) {
      const int chunk = tid + c * 256;
      const int row = chunk >> 3, col8 = chunk & 7;
      *reinterpret_cast<uint4*>(&xs[buf][row * kXsPitch + col8 * 8]) = xreg[c];
    }
  };

  // half step: octets J0, J0+1 of the current tile against LDS buffer `buf`.  All operand
  // reads of a 32-column step are issued before its first MFMA, so that LDS latency is
  // paid once per step and not once per activation tile.
  auto half_step = [&](int buf, auto j0tag) {
    constexpr int J0 = decltype(j0tag)::value;
    auto k32 = [&](auto jtag) {
      constexpr int J = decltype(jtag)::value;
      constexpr int jj = J - J0;
      Frag aw[RBW];
#pragma unroll
      for (int rr = 0; rr < RBW; rr++) {
        const int gg = GROUP == 32 ? J : 0;
        _Float16 s1 = scur[rr][gg];
        if constexpr (!ZP) s1 = (_Float16)((float)s1 * (float)(1 << (8 - BITS)));
        const half2v sc = {s1, s1};
        half2v zr = {(_Float16)0.f, (_Float16)0.f};
        if constexpr (ZP) zr = half2v{zcur[rr][gg], zcur[rr][gg]};
#ifdef MATGPTQ_DEBUG_NODEQUANT
        aw[rr].u[0] = wcur[rr][0]; aw[rr].u[1] = wcur[rr][1 % BITS]; aw[rr].u[2] = wcur[rr][0] ^ J; aw[rr].u[3] = wcur[rr][1 % BITS];
        (void)sc; (void)zr;
#else
        dequant_octet<BITS, J, ZP>(wcur[rr], kc_unpack, zr, sc, aw[rr]);
#endif
      }
      // activation operands in groups of four tiles: their reads are in flight together
      constexpr int MG = MT < 4 ? MT : 4;
#pragma unroll
      for (int m0g = 0; m0g < MT; m0g += MG) {
        Frag b[MG];
#pragma unroll
        for (int i = 0; i < MG; i++)
          b[i].v = *reinterpret_cast<const uint4*>(&xs[buf][((m0g + i) * 16 + r16) * kXsPitch + jj * 32 + q * 8]);
#pragma unroll
        for (int i = 0; i < MG; i++) {
#pragma unroll
          for (int rr = 0; rr < RBW; rr++)
            acc[rr][m0g + i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aw[rr].h, b[i].h, acc[rr][m0g + i], 0, 0, 0);
        }
      }
    };
    k32(std::integral_constant<int, J0>{});
    k32(std::integral_constant<int, J0 + 1>{});
  };

  // prologue
  load_x(0);
  load_weights(wcur, scur, zcur, 0);
  store_x(0);
  __syncthreads();

  const int H = a.k_tiles * 2;
  for (int kb = 0; kb < a.k_tiles; kb++) {
    // first half of the tile
    load_x(2 * kb + 1);
    if (kb + 1 < a.k_tiles) load_weights(wnxt, snxt, znxt, kb + 1);
    half_step(0, std::integral_constant<int, 0>{});
    store_x(1);
    __syncthreads();
    // second half
    if (2 * kb + 2 < H) load_x(2 * kb + 2);
    half_step(1, std::integral_constant<int, 2>{});
    if (2 * kb + 2 < H) store_x(0);
    __syncthreads();
    if (kb + 1 < a.k_tiles) {
#pragma unroll
      for (int rr = 0; rr < RBW; rr++) {
#pragma unroll
        for (int i = 0; i < BITS; i++) wcur[rr][i] = wnxt[rr][i];
#pragma unroll
        for (int gg = 0; gg < GPT; gg++) { scur[rr][gg] = snxt[rr][gg]; zcur[rr][gg] = znxt[rr][gg]; }
      }
    }
  }

  // epilogue: lane holds rows (weight rows) 4q..4q+3 of column (batch row) r16
#pragma unroll
  for (int rr = 0; rr < RBW; rr++) {
    const int rb = rb_first + rr;
    if (rb >= a.row_blocks) continue;
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
      const int m = m0 + mt * 16 + r16;
      if (m < a.M) {
        H4 o;
#pragma unroll
        for (int i = 0; i < 4; i++) o.h[i] = (_Float16)acc[rr][mt][i];
        *reinterpret_cast<uint2*>(a.y + (size_t)m * a.N + (size_t)rb * 16 + 4 * q) = o.v;
      }
    }
  }
}

template <int GROUP, bool ZP, int RBW, int MT>
hipError_t launch_cfg(const GemmArgs& a, hipStream_t stream) {
  const int n_tiles = (a.row_blocks + 4 * RBW - 1) / (4 * RBW);
  const int m_tiles = (a.M + 16 * MT - 1) / (16 * MT);
  const dim3 grid(n_tiles * m_tiles), block(256);
  hipLaunchKernelGGL((prefill_kernel<kBits, GROUP, ZP, RBW, MT>), grid, block, 0, stream, a,
                     n_tiles, m_tiles);
  return hipGetLastError();
}

template <int GROUP, bool ZP>
hipError_t launch_shape(const GemmArgs& a, int cfg, hipStream_t s) {
  switch (cfg) {
    case 0: return launch_cfg<GROUP, ZP, 4, 8>(a, s);   // 128 x 256
    case 1: return launch_cfg<GROUP, ZP, 8, 8>(a, s);   // 128 x 512
    case 2: return launch_cfg<GROUP, ZP, 4, 4>(a, s);   // 64 x 256
    case 3: return launch_cfg<GROUP, ZP, 2, 8>(a, s);   // 128 x 128
    case 4: return launch_cfg<GROUP, ZP, 2, 2>(a, s);   // 32 x 128
    case 5: return launch_cfg<GROUP, ZP, 8, 4>(a, s);   // 64 x 512
    case 6: return launch_cfg<GROUP, ZP, 8, 2>(a, s);   // 32 x 512
    default: return launch_cfg<GROUP, ZP, 4, 2>(a, s);  // 32 x 256
  }
}

}  // namespace

#define MATGPTQ_CAT2(a, b) a##b
#define MATGPTQ_CAT(a, b) MATGPTQ_CAT2(a, b)
// cfg selects the workgroup tile (see launch_shape).
hipError_t MATGPTQ_CAT(launch_prefill_b, MATGPTQ_BITS)(const GemmArgs& a, int group_size, int cfg,
                                                       hipStream_t stream) {
  const bool zp = a.zeros != nullptr;
  if (group_size == 128)
    return zp ? launch_shape<128, true>(a, cfg, stream) : launch_shape<128, false>(a, cfg, stream);
  if (group_size == 32)
    return zp ? launch_shape<32, true>(a, cfg, stream) : launch_shape<32, false>(a, cfg, stream);
  return zp ? launch_shape<-1, true>(a, cfg, stream) : launch_shape<-1, false>(a, cfg, stream);
}

}  // namespace matgptq
