// Prefill-regime kernel (M > 16): dense contraction on the matrix cores.
// Compiled once per bitwidth with -DMATGPTQ_BITS=b.  The reference has no kernel
// of this kind: its tensor-core path re-reads and re-dequantises every weight
// once per eight batch rows (inference_lib/matgptq_cuda/csrc/matgptq_gemm.cu:337-634,961-963).
//
//  * a workgroup of four waves owns TM = 16*MT activation rows and 64*RBW weight
//    rows; wave w owns the RBW row blocks [w*RBW, +RBW) of that range, so every
//    packed code is dequantised by exactly one wave, straight from registers into
//    the 16x32 MFMA operand (see dequant_pair for the arithmetic);
//  * the 128 x 256 tile (RBW 4, MT 8: the default for large batches) and the 128 x 128 tile
//    (RBW 2, MT 8) run two waves per SIMD with a ring loop.  The accumulators of the larger one
//    take half of a wave's 256 registers, so the activations never pass
//    through registers: buffer_load ... lds copies them into a ring of four unpadded LDS
//    buffers of 64 columns, three half tiles ahead, with an XOR swizzle of the 16-byte chunks
//    against bank conflicts and hand-counted vmcnt waits in front of the workgroup barriers.
//    One wave dequantises while the other wave of the SIMD multiplies.  Where such tiles number
//    no more than the CUs (batches of a few hundred rows), a workgroup of eight waves runs K in
//    two halves on one tile, each group of four waves with a ring of its own, and adds the two
//    sets of sums through LDS at the end: two waves per SIMD again, without a second workgroup;
//  * the other tiles stage the activations through registers into two padded LDS buffers
//    (global loads eight 32-column steps ahead, four for the largest tile) and pipeline inside
//    a wave: while the matrix cores work on one 32-column step, the vector ALU dequantises the
//    next step's weights (sched_group_barrier asks the compiler for that interleaving);
//  * in every loop an activation operand register is refilled from LDS as soon as the MFMAs
//    that read it have been issued, every global load is branch-free (tiles beyond K or N go
//    through a zero-length buffer descriptor), and scales and zeros stay in registers as
//    loaded (converted at use), so that nothing waits on a load right after issuing it;
//  * bf16 storage runs the same loops on the bf16 matrix instruction: the activations stay as
//    stored, the weights are formed in fp32 and rounded to bf16 once (see dequant_pair_bf16);
//  * fp32 accumulators live in registers for the whole K loop; the epilogue packs
//    four consecutive output columns per lane into one 8-byte store.
//
// Measured on this target: a loop of nothing but independent MFMAs reaches 1.37 PFLOP/s with
// one wave per SIMD and 1.91 PFLOP/s with two (nominal 2.5), which is why the default tile is
// sized for two resident waves per SIMD.
//
// Workgroup ids of the staged tiles are remapped so that the workgroups of one XCD (ids
// congruent modulo 8) walk consecutive activation tiles of the same weight rows and share
// those rows in their L2; the ring tile keeps the plain order.
#include "device_common.h"
#include "prefill_plan.h"

// (m0 in the clobber list of the LDS copies below: reserved, but the compiler keeps nothing in it)
#pragma clang diagnostic ignored "-Winline-asm"

#ifndef MATGPTQ_BITS
#error "compile with -DMATGPTQ_BITS={2,3,4,6,8}"
#endif

namespace matgptq {

namespace {

constexpr int kBits = MATGPTQ_BITS;
constexpr int kXs = 64;          // activation columns per LDS stage
#ifndef MATGPTQ_XPAD
#define MATGPTQ_XPAD 8
#endif
constexpr int kXsPitch = kXs + MATGPTQ_XPAD;  // halves per LDS row

// Two waves per SIMD (256 registers each) whenever the accumulators leave room for the rest:
// one wave alone cannot keep the matrix pipe busy.  The tile whose accumulators take half of
// that budget runs the ring loop below (activations straight into LDS, one operand set).
// (64 batch rows x 128 weight rows run the same loop: the K-split tile of batches whose 128-row tiles
// would leave half of the CUs idle)
constexpr bool prefill_lean(int rbw, int mt) {
  return ((rbw == 4 || rbw == 3 || rbw == 2) && mt == 8) || (rbw == 2 && mt == 4);
}
constexpr int prefill_min_waves(int rbw, int mt) { return rbw * mt * 4 < 128 || prefill_lean(rbw, mt) ? 2 : 1; }

// LDS of a workgroup, in halves: the ring loop keeps four unpadded buffers of 64 columns, the
// staged loops two padded ones.
constexpr int prefill_lds_halves(int rbw, int mt) {
  return prefill_lean(rbw, mt) ? 4 * 16 * mt * kXs : 2 * 16 * mt * kXsPitch;
}

// Wide codes on the 128 x 256 tile: two register sets of 6-bit codes (or of 8-bit codes next to
// zero points) for four row blocks do not fit beside the 128 accumulators.  Those formats keep ONE
// set and refill the words of an octet with the next tile's right after the octet has been
// dequantised (three 32-column steps before they are needed again), one small load per octet.
constexpr bool prefill_streams_codes(int bits, bool zp, int rbw, int mt) {
  (void)zp;
  return rbw == 4 && mt == 8 && (bits == 6 || bits == 8);
}
// loads refill_octet issues for octet j
constexpr int refill_loads(int bits, int j) { return bits == 6 && (j & 1) ? 2 : 1; }

// The words octet J of a lane is decoded from, out of the tile at `tile_off` (8 bits: words 2J, 2J+1;
// 6 bits: word J and, behind the odd octets, the word of low bits they share with their neighbour).
template <int BITS, int J>
__device__ __forceinline__ void refill_octet(BufRsrc rs, uint32_t tile_off, int lane, uint32_t (&w)[BITS]) {
  static_assert(BITS == 6 || BITS == 8, "wide codes only");
  if constexpr (BITS == 8) {
    const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rs, (J >> 1) * 1024 + lane * 16 + (J & 1) * 8, tile_off, 0);
    w[2 * J] = v.x;
    w[2 * J + 1] = v.y;
  } else {
    w[J] = __builtin_amdgcn_raw_buffer_load_b32(rs, lane * 16 + J * 4, tile_off, 0);
    if constexpr ((J & 1) != 0)
      w[4 + (J >> 1)] = __builtin_amdgcn_raw_buffer_load_b32(rs, 1024 + lane * 8 + (J >> 1) * 4, tile_off, 0);
  }
}

// One workgroup tile: activation rows [mtile * 16 MT, +16 MT) x the weight rows of the row blocks
// rb_base + [nt * 4 RBW, +4 RBW), where lid = nt * m_tiles + mtile.  `lds` is the workgroup's
// LDS (KS * prefill_lds_halves(RBW, MT) halves, 16-byte aligned).
// KS = 2 (ring tiles only): a workgroup of eight waves, two groups of four that each walk one
// half of K on the same tile with a ring of their own, so that a layer whose tiles number no more
// than the CUs still runs two waves per SIMD; the second group's sums pass through LDS at the end.
// PAIR (ring tiles only): a workgroup of eight waves again, but each group of four owns a tile of its
// own (tiles 2 lid and 2 lid + 1, the whole of K, a ring each): two plain workgroups in one, for
// kernels whose other workgroups need eight waves.  A tile index from `lid_limit` on is empty.
template <int BITS, int GROUP, bool ZP, int RBW, int MT, int KS = 1, bool PAIR = false>
__device__ __forceinline__ void prefill_body(const GemmArgs& a, int lid, int m_tiles, int rb_base,
                                             _Float16* lds, int lid_limit = 0x7fffffff) {
  static_assert(KS == 1 || (KS == 2 && prefill_lean(RBW, MT)), "K is split inside the ring tiles only");
  static_assert(!PAIR || (KS == 1 && prefill_lean(RBW, MT)), "paired tiles are ring tiles with the whole of K each");
  constexpr int TM = 16 * MT;
  constexpr int GPT = GROUP == 32 ? 4 : 1;
  constexpr int XCHUNKS = TM * (kXs / 8) / 256;  // 16-byte chunks per thread per stage
  static_assert(TM * (kXs / 8) % 256 == 0, "activation tile must split evenly over 256 threads");
  constexpr int kXsBuf = TM * kXsPitch;  // halves per buffer of the staged loops
  _Float16* const xs = lds;              // [2][kXsBuf] (unused by the ring loop)

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave_wg = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: tile offsets stay scalar
  const int wave = wave_wg & 3;  // within its group of four
  const int grp = KS == 1 && !PAIR ? 0 : ((wave_wg >> 2) & 1);
  if constexpr (PAIR) lid = 2 * lid + grp;
  // K tiles [k_lo, k_hi) in kt_n trips (the same count for both groups: they share the barriers; a
  // tile beyond k_hi reads as zeros)
  const int kt_n = KS == 1 ? a.k_tiles : (a.k_tiles + 1) / 2;
  const int k_lo = KS == 1 ? 0 : grp * kt_n;
  const int k_hi = KS == 1 || grp == 1 ? a.k_tiles : kt_n;
  lds += grp * prefill_lds_halves(RBW, MT);
  const int r16 = lane & 15;
  const int q = lane >> 4;

  const int nt = lid / m_tiles;
  const int mtile = lid - nt * m_tiles;
  const int m0 = mtile * TM;
  // (an empty tile: every row block out of range, so nothing is fetched and nothing stored)
  const int rb_first = lid < lid_limit ? rb_base + (nt * 4 + wave) * RBW : a.row_blocks;

  constexpr uint32_t tile_bytes = (uint32_t)tile_words(BITS) * 4;
  const uint32_t rb_bytes = (uint32_t)a.k_tiles * tile_bytes;
  const uint32_t w_bytes = (uint32_t)a.row_blocks * rb_bytes;
  const uint32_t aux_bytes = (uint32_t)a.row_blocks * a.G * 32;  // scales / zeros: [N/16][G][16] halves

  float4v acc[RBW][MT];
#pragma unroll
  for (int rr = 0; rr < RBW; rr++)
#pragma unroll
    for (int mt = 0; mt < MT; mt++) acc[rr][mt] = float4v{0.f, 0.f, 0.f, 0.f};

  const UnpackConsts<BITS> kc_unpack;
  const float kc_zero = __uint_as_float(opaque_vgpr(0u));  // a zero the optimiser cannot see through
  uint32_t wcur[RBW][BITS], wnxt[RBW][BITS];
  // scales and zeros as loaded (16 bits in a register each): converted where they are used, so
  // that nothing has to wait for these loads right after they are issued
  uint32_t scur[RBW][GPT], snxt[RBW][GPT];
  uint32_t zcur[RBW][GPT], znxt[RBW][GPT];

  // Branch-free loads: a tile beyond K, or a row block beyond N, is read through a
  // descriptor of zero length (every lane out of range: zeros come back, nothing is fetched).
  auto load_weights = [&](uint32_t (&w)[RBW][BITS], uint32_t (&s)[RBW][GPT], uint32_t (&z)[RBW][GPT],
                          int trip) {
    const int kb = trip + k_lo;
#pragma unroll
    for (int rr = 0; rr < RBW; rr++) {
      const int rb = rb_first + rr;
      const bool valid = rb < a.row_blocks && kb < k_hi;
      const BufRsrc wr = make_rsrc(a.packed, valid ? w_bytes : 0u);
      const BufRsrc sr = make_rsrc(a.scales, valid ? aux_bytes : 0u);
      const BufRsrc zr = make_rsrc(ZP ? a.zeros : a.scales, valid ? aux_bytes : 0u);
      load_tile_words<BITS, 0>(wr, (uint32_t)rb * rb_bytes + (uint32_t)kb * tile_bytes, lane, w[rr]);
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

  // Activation tile: two register sets, one per LDS buffer; a set is loaded four steps
  // before it is stored.  Rows beyond M fall outside the descriptor and read as zero.
  const uint32_t x_bytes = (uint32_t)a.M * (uint32_t)a.K * 2u;
  uint32_t x_voff[XCHUNKS], x_lds[XCHUNKS];
#pragma unroll
  for (int c = 0; c < XCHUNKS; c++) {
    const int chunk = tid + c * 256;
    const int row = chunk >> 3, col8 = chunk & 7;
    const uint32_t m = (uint32_t)(m0 + row);
    x_voff[c] = m < (uint32_t)a.M ? (m * (uint32_t)a.K + col8 * 8) * 2u : x_bytes;
    x_lds[c] = (uint32_t)(row * kXsPitch + col8 * 8);
  }
  auto load_x = [&](u32x4 (&xr)[XCHUNKS], int h) {  // columns [h*64, +64)
    const bool valid = h < 2 * a.k_tiles;
    const BufRsrc xres = make_rsrc(a.x, valid ? x_bytes : 0u);
#pragma unroll
    for (int c = 0; c < XCHUNKS; c++)
      xr[c] = __builtin_amdgcn_raw_buffer_load_b128(xres, x_voff[c], (uint32_t)h * (kXs * 2), 0);
    __builtin_amdgcn_sched_barrier(0);
  };
  auto store_x = [&](const u32x4 (&xr)[XCHUNKS], int buf) {
#pragma unroll
    for (int c = 0; c < XCHUNKS; c++)
      *reinterpret_cast<u32x4*>(&xs[buf * kXsBuf + x_lds[c]]) = xr[c];  // as stored: fp16 or bf16
  };

  auto dequant_step = [&](Frag (&aw)[RBW], const uint32_t (&w)[RBW][BITS], const uint32_t (&s)[RBW][GPT],
                          const uint32_t (&z)[RBW][GPT], auto jtag) {
    constexpr int J = decltype(jtag)::value;
#pragma unroll
    for (int rr = 0; rr < RBW; rr++) {
      const int gg = GROUP == 32 ? J : 0;
      if constexpr (kBf16) {
        // bf16 storage: scale * 2^(8-b) and scale * (zero - 128) in fp32, weights for the bf16 MFMA
        const float s0 = bf16_bits_to_float(s[rr][gg]);
        const float sm = s0 * (float)(1 << (8 - BITS));
        float sz = kc_zero;
        if constexpr (ZP) sz = s0 * (bf16_bits_to_float(z[rr][gg]) - 128.0f);
        dequant_octet_bf16<BITS, J>(w[rr], kc_unpack, sm, sz, aw[rr]);
      } else {
        // fp16 storage: scale * 2^(8-b) and scale * (zero - 128)
        const _Float16 s0 = __builtin_bit_cast(_Float16, (uint16_t)s[rr][gg]);
        const _Float16 s1 = (_Float16)((float)s0 * (float)(1 << (8 - BITS)));  // scale * m
        _Float16 z1 = (_Float16)0.f;
        if constexpr (ZP) z1 = s0 * (__builtin_bit_cast(_Float16, (uint16_t)z[rr][gg]) - (_Float16)128.0f);
        const half2v sc = {s1, s1};
        const half2v zr = {z1, z1};
        dequant_octet<BITS, J, ZP>(w[rr], kc_unpack, zr, sc, aw[rr]);
      }
    }
  };
  // one MFMA 16x16x32 in the storage type: weights and activations are both fp16, or both bf16
  auto mma = [](const Frag& wa, const Frag& xb, float4v c) {
    if constexpr (kBf16)
      return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wa.h), __builtin_bit_cast(bf16x8, xb.h),
                                                     c, 0, 0, 0);
    else
      return __builtin_amdgcn_mfma_f32_16x16x32_f16(wa.h, xb.h, c, 0, 0, 0);
  };
  auto read_frag = [&](Frag& b, int i, int buf, int jj) {
    b.v = *reinterpret_cast<const uint4*>(&xs[buf * kXsBuf + (i * 16 + r16) * kXsPitch + jj * 32 + q * 8]);
  };
  // One 32-column step of the software pipeline: the matrix cores multiply `aw` by the
  // activation operands `b`; as soon as the MFMAs that use b[i] have been issued, b[i] is
  // refilled with the operand of the next step (LDS buffer `nbuf`, columns [njj*32, +32)),
  // and the vector ALU dequantises the next step's weights (`next()`) in between.  The
  // scheduling groups ask for a few vector instructions and one LDS read after every RBW MFMAs.
  auto step = [&](const Frag (&aw)[RBW], Frag (&b)[MT], int nbuf, int njj, auto&& next) {
    next();
#pragma unroll
    for (int i = 0; i < MT; i++) {
#pragma unroll
      for (int rr = 0; rr < RBW; rr++)
        acc[rr][i] = mma(aw[rr], b[i], acc[rr][i]);
      read_frag(b[i], i, nbuf, njj);
    }
    constexpr int kValuPerMfma = (RBW * 24 + RBW * MT - 1) / (RBW * MT);
#pragma unroll
    for (int i = 0; i < MT; i++) {
#pragma unroll
      for (int rr = 0; rr < RBW; rr++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);             // MFMA
        __builtin_amdgcn_sched_group_barrier(0x002, kValuPerMfma, 0);  // VALU
      }
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // DS read
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  if constexpr (prefill_lean(RBW, MT)) {
    // The 128 x 256 tile at two waves per SIMD: its accumulators take half of the wave's 256
    // registers, so the activations never pass through registers.  buffer_load ... lds copies
    // them from global memory straight into a ring of four LDS buffers (one half tile of 64
    // columns each, 128 rows of 128 bytes, no padding), three half tiles ahead of their use.
    // A wave copies 8 rows per instruction (lane l: row l/8, 16-byte chunk l%8 of the LDS
    // row); chunk c of LDS row r holds columns 8*(c ^ ((r>>1)&7)) of the half tile, so the
    // sixteen lanes of an operand read (rows r..r+15, one column chunk) hit sixteen different
    // 16-byte bank groups.  The waits for these copies are written by hand: vmcnt counts every
    // buffer load of the wave in issue order, and each wait below names how many younger ones
    // may still be in flight (see the issue order at the loop).
    _Float16* const ring0 = lds;
    _Float16* const ring1 = lds + TM * kXs;
    _Float16* const ring2 = lds + 2 * TM * kXs;
    _Float16* const ring3 = lds + 3 * TM * kXs;
    static_assert(TM % 32 == 0, "a wave copies a quarter of the rows, eight per instruction");
    constexpr int kRowsPerWave = TM / 4;
    constexpr int kD = kRowsPerWave / 8;  // copy instructions of a wave per half tile
    // this lane's part of a copy: rows wave*kRowsPerWave + i*8 + lane/8, LDS chunk lane%8
    static_assert(kD <= 4, "offsets of at most four copies are kept");
    uint32_t dma_voff[4];  // kD of them in use (a bound that depends on the tile does not pass the host compilation)
#pragma unroll
    for (int i = 0; i < kD; i++) {
      const int r = wave * kRowsPerWave + i * 8 + (lane >> 3);
      const int c = (lane & 7) ^ ((r >> 1) & 7);
      const uint32_t m = (uint32_t)(m0 + r);
      dma_voff[i] = m < (uint32_t)a.M ? (m * (uint32_t)a.K + c * 8) * 2u : x_bytes;
    }
    auto dma = [&](_Float16* ring, int step) {  // half tile `step` of the walk into `ring`
      const int ih = step + 2 * k_lo;
      const bool valid = ih < 2 * k_hi;
      const BufRsrc xres = make_rsrc(a.x, valid ? x_bytes : 0u);
      if constexpr (KS == 2 && RBW < 4) {
        // The narrower tiles with K split in the workgroup issue the copies as assembly text.  The compiler places its own
        // counter waits in front of LDS reads that may overlap a copy in flight and, on loop paths that
        // are never taken, in front of the first use of the weights; it cannot tell the ring buffers
        // apart, so these waits let nothing stay in flight.  A wave that stalls there holds up both
        // groups at the next barrier.  Copies it does not see leave only the hand-counted waits, which
        // every LDS read of copied data already sits behind; its own waits for register loads count
        // fewer loads than are in flight and stay on the safe side.  (Measured at 4 bits: 128 x 128 and
        // 128 x 192 tiles with K split 2 to 10 % faster; the 128 x 256 tile 1 to 2 % slower with K split,
        // no difference in pairs or in workgroups of four waves: those keep the intrinsic.)
        const uint64_t xa = (uint64_t)(uintptr_t)a.x;
        const u32x4 xd = {(uint32_t)xa, (uint32_t)(xa >> 32) & 0xffffu, valid ? x_bytes : 0u, 0x00020000u};
        const uint32_t base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)(ring + wave * kRowsPerWave * kXs);
#pragma unroll
        for (int i = 0; i < kD; i++)  // m0: LDS address of the wave's 8 rows; one wait state before its use
          asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                       :
                       : "s"(base + i * 8 * kXs * 2), "v"(dma_voff[i]), "s"(xd), "s"((uint32_t)ih * (kXs * 2))
                       : "memory", "m0");
      } else {
#pragma unroll
        for (int i = 0; i < kD; i++)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(
              xres, (__attribute__((address_space(3))) void*)(ring + (wave * kRowsPerWave + i * 8) * kXs), 16, dma_voff[i],
              (uint32_t)ih * (kXs * 2), 0, 0);
      }
    };
    // operand read: row i*16 + r16, columns [jj*32 + q*8, +8)
    const int sw = (r16 >> 1) & 7;
    const int frag_off[2] = {r16 * kXs + ((q ^ sw) * 8), r16 * kXs + (((4 + q) ^ sw) * 8)};
    auto ring_frag = [&](Frag& bv, const _Float16* ring, int i, int jj) {
      bv.v = *reinterpret_cast<const uint4*>(ring + i * 16 * kXs + frag_off[jj]);
    };
    // wait until at most `n` buffer loads of this wave are in flight, then meet the workgroup
    auto wait_and_meet = [&](auto ntag) {
      // (the counter holds 63 at most: with more younger loads than that, 63 still excludes the
      // one waited for)
      constexpr int n = decltype(ntag)::value < 63 ? decltype(ntag)::value : 63;
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_waitcnt((n & 15) | (7 << 4) | (0 << 8) | ((n >> 4) << 14));  // vmcnt(n), lgkmcnt(0)
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
    };
    // one 32-column step: dequantise octet J of the tile into `aw`, multiply by the operands in
    // `bv`, and refill each bv[i] for the next step (ring `nring`, columns [njj*32, +32)) as soon
    // as its MFMAs are issued.  Two waves share a SIMD: one's vector work overlaps the other's
    // matrix work, which is why a single operand set is enough.
    Frag aw[RBW];
    Frag bv[MT];
    constexpr bool kReloadBehindBranch = GROUP != 32;  // see the loops below
    auto dstep = [&](const uint32_t (&w)[RBW][BITS], const uint32_t (&sv)[RBW][GPT], const uint32_t (&zv)[RBW][GPT],
                     auto jtag, const _Float16* nring, int njj) {
      dequant_step(aw, w, sv, zv, jtag);
      // two halves of two row blocks each: the vector work of the second half can be issued
      // between the MFMAs of the first; the operands are refilled behind the second half
      // Workgroups of eight waves: the wave that has its operands ready issues its MFMAs ahead of the
      // vector work of the SIMD's other wave (measured at 4 bits: K split 1.5 to 4.5 % faster, pairs
      // with a split tail 1.3 %; no difference in workgroups of four waves, which go without)
      if constexpr (KS == 2 || PAIR) __builtin_amdgcn_s_setprio(1);
#pragma unroll
      for (int i = 0; i < MT; i++) {
#pragma unroll
        for (int rr = 0; rr < RBW / 2; rr++)
          acc[rr][i] = mma(aw[rr], bv[i], acc[rr][i]);
      }
#pragma unroll
      for (int i = 0; i < MT; i++) {
#pragma unroll
        for (int rr = RBW / 2; rr < RBW; rr++)
          acc[rr][i] = mma(aw[rr], bv[i], acc[rr][i]);
        ring_frag(bv[i], nring, i, njj);
      }
      if constexpr (KS == 2 || PAIR) __builtin_amdgcn_s_setprio(0);
      constexpr int kHalf = (RBW / 2) * MT;              // MFMAs of the first half
      constexpr int kRest = (RBW - RBW / 2) * MT;        // ... of the second (one more row block when RBW is odd)
      constexpr int kValuHalf = (RBW / 2) * 26;          // vector instructions of the first half's row blocks, roughly
      constexpr int kValuRest = (RBW - RBW / 2) * 26;
      // The ordering hints pay 1 % at 2, 3 and 4 bits.  The wide codes go without: 6-bit codes spill
      // with them (88 registers on the 128 x 256 tile), 8-bit codes run 0 to 2 % faster left alone.
#ifndef MATGPTQ_NO_GROUPS
      if constexpr (BITS != 6 && BITS != 8) {
      __builtin_amdgcn_sched_group_barrier(0x002, kValuHalf, 0);
#pragma unroll
      for (int n = 0; n < kHalf; n++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, (kValuRest + kHalf - 1) / kHalf, 0);
      }
#pragma unroll
      for (int n = 0; n < kRest; n++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if (n & 1) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      }
#endif
      __builtin_amdgcn_sched_barrier(0);
    };
    using J0 = std::integral_constant<int, 0>;
    using J1 = std::integral_constant<int, 1>;
    using J2 = std::integral_constant<int, 2>;
    using J3 = std::integral_constant<int, 3>;
    if constexpr (prefill_streams_codes(BITS, ZP, RBW, MT)) {
      // ---- one set of codes, refilled octet by octet; scales and zeros keep their two sets ----
      // loads per refill of octet J for all row blocks, and per set of scales (and zeros)
      constexpr int r0 = RBW * refill_loads(BITS, 0), r1 = RBW * refill_loads(BITS, 1);
      constexpr int r2 = RBW * refill_loads(BITS, 2), r3 = RBW * refill_loads(BITS, 3);
      constexpr int kS = RBW * GPT * (ZP ? 2 : 1);
      auto refill = [&](auto jtag, int trip) {  // octet J of the tile of that trip into the one set of codes
        constexpr int J = decltype(jtag)::value;
        const int kb = trip + k_lo;
#pragma unroll
        for (int rr = 0; rr < RBW; rr++) {
          const int rb = rb_first + rr;
          const bool valid = rb < a.row_blocks && kb < k_hi;
          const BufRsrc wr = make_rsrc(a.packed, valid ? w_bytes : 0u);
          refill_octet<BITS, J>(wr, (uint32_t)rb * rb_bytes + (uint32_t)kb * tile_bytes, lane, wcur[rr]);
        }
        __builtin_amdgcn_sched_barrier(0);
      };
      auto load_aux = [&](uint32_t (&sv)[RBW][GPT], uint32_t (&zv)[RBW][GPT], int trip) {
        const int kb = trip + k_lo;
#pragma unroll
        for (int rr = 0; rr < RBW; rr++) {
          const int rb = rb_first + rr;
          const bool valid = rb < a.row_blocks && kb < k_hi;
          const BufRsrc sr = make_rsrc(a.scales, valid ? aux_bytes : 0u);
          const BufRsrc zr = make_rsrc(ZP ? a.zeros : a.scales, valid ? aux_bytes : 0u);
#pragma unroll
          for (int gg = 0; gg < GPT; gg++) {
            const uint32_t g = GROUP == -1 ? 0u : (uint32_t)kb * GPT + gg;
            const uint32_t so = ((uint32_t)rb * a.G + g) * 32;
            sv[rr][gg] = __builtin_amdgcn_raw_buffer_load_b16(sr, r16 * 2, so, 0);
            if constexpr (ZP) zv[rr][gg] = __builtin_amdgcn_raw_buffer_load_b16(zr, r16 * 2, so, 0);
            else zv[rr][gg] = 0u;
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      };
      // Issue order of the wave's buffer loads (D = 4 copies of a half tile, Rj = refill of octet j,
      // S = scales and zeros of a tile):
      //   prologue  D0 D1 D2 D3  R0(0) R1(0) R2(0) R3(0)  S(0) S(1)
      //   tile t    [octet 0] R0(t+1) | barrier A, D(2t+4) | [1] R1(t+1) [2] R2(t+1) | barrier B, D(2t+5) |
      //             [3] R3(t+1) S(t+2)
      // Barrier A of tile t needs D(2t+1), issued behind barrier B of tile t-2; issued after it:
      //   R3 S | R0 D R1 R2 D R3 S | R0, and at t = 0 (D1 from the prologue): D2 D3 R0..R3 S S | R0, which is
      //   r3 loads fewer: the smaller count is used for every tile (a stricter wait, on loads that are
      //   more than a tile old).  Barrier B of tile t needs D(2t+2), issued behind barrier A of tile t-1;
      //   issued after it: R1 R2 D R3 S | R0 D R1 R2 (more at t = 0).
      constexpr int kWaitA = 2 * kD + 2 * r0 + r1 + r2 + r3 + 2 * kS;
      constexpr int kWaitB = 2 * kD + r0 + 2 * r1 + 2 * r2 + r3 + kS;
      dma(ring0, 0);
      dma(ring1, 1);
      dma(ring2, 2);
      dma(ring3, 3);
      refill(J0{}, 0);
      refill(J1{}, 0);
      refill(J2{}, 0);
      refill(J3{}, 0);
      load_aux(scur, zcur, 0);
      load_aux(snxt, znxt, 1);
      wait_and_meet(std::integral_constant<int, 3 * kD + r0 + r1 + r2 + r3 + 2 * kS>{});  // D0 has landed
#pragma unroll
      for (int i = 0; i < MT; i++) ring_frag(bv[i], ring0, i, 0);
      auto stile = [&](int kb, uint32_t (&sc)[RBW][GPT], uint32_t (&zc)[RBW][GPT], _Float16* ra, _Float16* rb,
                       _Float16* rn) {
        dstep(wcur, sc, zc, J0{}, ra, 1);
        refill(J0{}, kb + 1);
        wait_and_meet(std::integral_constant<int, kWaitA>{});
        dma(ra, 2 * kb + 4);
        dstep(wcur, sc, zc, J1{}, rb, 0);
        refill(J1{}, kb + 1);
        dstep(wcur, sc, zc, J2{}, rb, 1);
        refill(J2{}, kb + 1);
        wait_and_meet(std::integral_constant<int, kWaitB>{});
        dma(rb, 2 * kb + 5);
        dstep(wcur, sc, zc, J3{}, rn, 0);
        refill(J3{}, kb + 1);
      };
      // (S(t+2), into the set that tile t has just left, is issued behind the branch: see the loop below)
      for (int kb = 0; kb < kt_n; kb += 2) {
        stile(kb, scur, zcur, ring0, ring1, ring2);
        if constexpr (!kReloadBehindBranch) load_aux(scur, zcur, kb + 2);
        if (kb + 1 < kt_n) {
          if constexpr (kReloadBehindBranch) load_aux(scur, zcur, kb + 2);
          stile(kb + 1, snxt, znxt, ring2, ring3, ring0);
          load_aux(snxt, znxt, kb + 3);
        }
      }
    } else {
    // buffer loads one load_weights() issues: the codes, then a scale (and a zero) per group
      constexpr int kW = RBW * tile_load_count(BITS) + RBW * GPT * (ZP ? 2 : 1);
      // issue order of the wave's buffer loads: prologue  D0 D1 D2 D3 W0 W1 ; then per tile t
      //   after the first barrier D(2t+4), after the second barrier D(2t+5), at its end W(t+2)
      // (D = 4 copies of one half tile, W = kW loads of one tile's codes, scales and zeros)
      dma(ring0, 0);
      dma(ring1, 1);
      dma(ring2, 2);
      dma(ring3, 3);
      load_weights(wcur, scur, zcur, 0);
      load_weights(wnxt, snxt, znxt, 1);
      wait_and_meet(std::integral_constant<int, 3 * kD + 2 * kW>{});  // D0 has landed
  #pragma unroll
      for (int i = 0; i < MT; i++) ring_frag(bv[i], ring0, i, 0);
      // one tile; ra / rb: the rings of its two half tiles, rn: the ring of the next tile's first
      // (measured and not adopted: one barrier per tile, in front of its last step, with the tile after
      // next requested into both rings behind it - 1.5 to 2 % slower at M = 2048 on every layer)
      auto dtile = [&](int kb, uint32_t (&wc)[RBW][BITS], uint32_t (&sc)[RBW][GPT], uint32_t (&zc)[RBW][GPT],
                       _Float16* ra, _Float16* rb, _Float16* rn) {
        dstep(wc, sc, zc, J0{}, ra, 1);
        // needs D(2kb+1); younger in steady state: W(kb) D(2kb+2) D(2kb+3) W(kb+1)
        wait_and_meet(std::integral_constant<int, 2 * kD + 2 * kW>{});
        dma(ra, 2 * kb + 4);  // every wave is past its reads of ra
        dstep(wc, sc, zc, J1{}, rb, 0);
        dstep(wc, sc, zc, J2{}, rb, 1);
        // needs D(2kb+2); younger: D(2kb+3) W(kb+1) D(2kb+4)
        wait_and_meet(std::integral_constant<int, 2 * kD + kW>{});
        dma(rb, 2 * kb + 5);
        dstep(wc, sc, zc, J3{}, rn, 0);
      };
      // W(t+2) goes into the set that tile t has just left.  The first tile's set is reloaded behind
      // the branch, not in front of it: the compiler places its own counter waits over every path of
      // the flow graph, and the path that skips the second tile leads from the end of the first
      // straight back to its start.  With the reload in front of the branch, the loads the top of the
      // loop needs would be the youngest ones on that path, and its waits would let nothing stay in
      // flight; on the path that is taken, a whole tile's loads are younger.  (Group size 32 keeps the
      // reload in front: with four scales and zeros per row block the registers are full, and the
      // other order spills.)
      for (int kb = 0; kb < kt_n; kb += 2) {
        dtile(kb, wcur, scur, zcur, ring0, ring1, ring2);
        if constexpr (!kReloadBehindBranch) load_weights(wcur, scur, zcur, kb + 2);
        if (kb + 1 < kt_n) {
          if constexpr (kReloadBehindBranch) load_weights(wcur, scur, zcur, kb + 2);
          dtile(kb + 1, wnxt, snxt, znxt, ring2, ring3, ring0);
          load_weights(wnxt, snxt, znxt, kb + 3);
        }
      }
    }
  } else {
  Frag awA[RBW], awB[RBW];
  Frag bf[MT];
  using J0 = std::integral_constant<int, 0>;
  using J1 = std::integral_constant<int, 1>;
  using J2 = std::integral_constant<int, 2>;
  using J3 = std::integral_constant<int, 3>;

  if constexpr (RBW * MT * 4 >= 256) {
    // the accumulators fill the accumulation registers: one tile per trip, activations two
    // half tiles ahead, weights one tile ahead
    u32x4 xo[2][XCHUNKS];
    // prologue: half 0 into buffer 0, halves 1 and 2 into the register sets
    load_x(xo[0], 0);
    load_weights(wcur, scur, zcur, 0);
    store_x(xo[0], 0);
    load_x(xo[0], 1);
    load_x(xo[1], 2);
    dequant_step(awA, wcur, scur, zcur, J0{});
    __syncthreads();
  #pragma unroll
    for (int i = 0; i < MT; i++) read_frag(bf[i], i, 0, 0);

    for (int kb = 0; kb < a.k_tiles; kb++) {
      load_weights(wnxt, snxt, znxt, kb + 1);
      step(awA, bf, 0, 1, [&] { dequant_step(awB, wcur, scur, zcur, J1{}); });
      store_x(xo[0], 1);  // buffer 1 was last read during step 2 of the previous tile
      load_x(xo[0], 2 * kb + 3);
      __syncthreads();
      step(awB, bf, 1, 0, [&] { dequant_step(awA, wcur, scur, zcur, J2{}); });
      step(awA, bf, 1, 1, [&] { dequant_step(awB, wcur, scur, zcur, J3{}); });
      store_x(xo[1], 0);  // buffer 0 was last read during step 0 of this tile
      load_x(xo[1], 2 * kb + 4);
      __syncthreads();
      // the last step of the tile prepares octet 0 of the next tile
      step(awB, bf, 0, 0, [&] { dequant_step(awA, wnxt, snxt, znxt, J0{}); });
  #pragma unroll
      for (int rr = 0; rr < RBW; rr++) {
  #pragma unroll
        for (int i = 0; i < BITS; i++) wcur[rr][i] = wnxt[rr][i];
  #pragma unroll
        for (int gg = 0; gg < GPT; gg++) { scur[rr][gg] = snxt[rr][gg]; zcur[rr][gg] = znxt[rr][gg]; }
      }
    }
  } else {
    // Register sets of the activation prefetch: half tile h travels in set h % NX and is
    // loaded NX half tiles (2 NX steps) before it is stored to LDS.  Weights: two sets (even
    // and odd tiles); a set is reloaded for the tile after next as soon as its last octet
    // has been dequantised, five steps before that tile's first octet is needed.
    constexpr int NX = 4;
    u32x4 xr[NX][XCHUNKS];
    load_x(xr[0], 0);
    load_weights(wcur, scur, zcur, 0);
    load_weights(wnxt, snxt, znxt, 1);
    store_x(xr[0], 0);
  #pragma unroll
    for (int h = 1; h <= NX; h++) load_x(xr[h & (NX - 1)], h);
    dequant_step(awA, wcur, scur, zcur, J0{});
    __syncthreads();
  #pragma unroll
    for (int i = 0; i < MT; i++) read_frag(bf[i], i, 0, 0);

    // one tile: weights `wc` (the next tile's are in `wn`), activation sets `sa` / `sb` for
    // the half tiles 2 kb + 1 (LDS buffer 1) and 2 kb + 2 (buffer 0)
    auto tile = [&](int kb, uint32_t (&wc)[RBW][BITS], uint32_t (&sc)[RBW][GPT], uint32_t (&zc)[RBW][GPT],
                    const uint32_t (&wn)[RBW][BITS], const uint32_t (&sn)[RBW][GPT],
                    const uint32_t (&zn)[RBW][GPT], u32x4 (&sa)[XCHUNKS], u32x4 (&sb)[XCHUNKS]) {
      step(awA, bf, 0, 1, [&] { dequant_step(awB, wc, sc, zc, J1{}); });
      store_x(sa, 1);  // buffer 1 was last read during step 2 of the previous tile
      load_x(sa, 2 * kb + 1 + NX);
      __syncthreads();
      step(awB, bf, 1, 0, [&] { dequant_step(awA, wc, sc, zc, J2{}); });
      step(awA, bf, 1, 1, [&] { dequant_step(awB, wc, sc, zc, J3{}); });
      load_weights(wc, sc, zc, kb + 2);  // this set is free now
      store_x(sb, 0);  // buffer 0 was last read during step 0 of this tile
      load_x(sb, 2 * kb + 2 + NX);
      __syncthreads();
      // the last step of the tile prepares octet 0 of the next tile
      step(awB, bf, 0, 0, [&] { dequant_step(awA, wn, sn, zn, J0{}); });
    };
    for (int kb = 0; kb < a.k_tiles; kb += 2) {
      tile(kb, wcur, scur, zcur, wnxt, snxt, znxt, xr[1 & (NX - 1)], xr[2 & (NX - 1)]);
      if (kb + 1 < a.k_tiles)
        tile(kb + 1, wnxt, snxt, znxt, wcur, scur, zcur, xr[3 & (NX - 1)], xr[4 & (NX - 1)]);
    }
  }

  }  // pipelined loop

  if constexpr (prefill_lean(RBW, MT)) {
    // Epilogue of the ring tiles through LDS, so that the output leaves in whole row segments: a
    // lane holds 4 consecutive output columns of one batch row per accumulator (8 bytes, 32 per
    // row and store), while all workgroups of a round write their tiles at the same time and
    // the memory system takes 16-byte pieces of full 128-byte (64-byte) row segments better.
    // The ring is free once every wave is past its last operand read and every copy into it
    // has landed (also the copies of half tiles beyond K, which write zeros).  A wave owns the
    // 128 x 16 RBW block of its row blocks: 16-byte chunk c of row r sits at chunk c ^ (r % CH).
    // (three row blocks: rows of eight chunks as well, the last two unused)
    constexpr int CH = RBW == 3 ? 8 : RBW * 2;  // 16-byte chunks per row of the block
    constexpr int ROWH = CH * 8;                // halves per row
    __builtin_amdgcn_s_waitcnt(0);     // vmcnt(0) expcnt(0) lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    _Float16* blk = lds + wave * (TM * ROWH);
    if constexpr (KS == 2) {
      // The second group hands its sums to the first as they lie in the registers (16 bytes per
      // lane): those of its first H row blocks through its own ring, the others through the part of
      // the first group's ring that wave `wave` of that group is about to use for its own output
      // block, so no wave writes where another still reads.
      constexpr int H = (RBW + 1) / 2;
      static_assert((RBW - H) * MT * 64 * 16 <= TM * ROWH * 2 && 4 * H * MT * 64 * 16 <= prefill_lds_halves(RBW, MT) * 2,
                    "the partial sums must fit the two rings");
      _Float16* const lds0 = lds - grp * prefill_lds_halves(RBW, MT);
      float4v* const p1 = reinterpret_cast<float4v*>(lds0 + prefill_lds_halves(RBW, MT)) + wave * (H * MT * 64) + lane;
      float4v* const p0 = reinterpret_cast<float4v*>(lds0 + wave * (TM * ROWH)) + lane;
      if (grp == 1) {
#pragma unroll
        for (int rr = 0; rr < RBW; rr++)
#pragma unroll
          for (int mt = 0; mt < MT; mt++)
            (rr < H ? p1[(rr * MT + mt) * 64] : p0[((rr - H) * MT + mt) * 64]) = acc[rr][mt];
      }
      __syncthreads();
      if (grp == 1) return;
#pragma unroll
      for (int rr = 0; rr < RBW; rr++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
          acc[rr][mt] += rr < H ? p1[(rr * MT + mt) * 64] : p0[((rr - H) * MT + mt) * 64];
    }
#pragma unroll
    for (int rr = 0; rr < RBW; rr++) {
#pragma unroll
      for (int mt = 0; mt < MT; mt++) {
        const int r = mt * 16 + r16;
        const int c = rr * 2 + (q >> 1);
        uint16_t o[4];
#pragma unroll
        for (int i = 0; i < 4; i++) o[i] = float_to_storage(acc[rr][mt][i]);
        *reinterpret_cast<uint2*>(blk + r * ROWH + ((c ^ (r & (CH - 1))) * 8) + (q & 1) * 4) =
            make_uint2((uint32_t)o[0] | ((uint32_t)o[1] << 16), (uint32_t)o[2] | ((uint32_t)o[3] << 16));
      }
    }
    constexpr int RPI = 64 / CH;  // rows per store instruction
    const int c = lane % CH;
    const int rb = rb_first + (c >> 1);
#pragma unroll
    for (int i = 0; i < TM / RPI; i++) {
      const int r = i * RPI + lane / CH;
      const int m = m0 + r;
      const uint4 v = *reinterpret_cast<const uint4*>(blk + r * ROWH + ((c ^ (r & (CH - 1))) * 8));
      if (m < a.M && rb < a.row_blocks && c < RBW * 2)
        *reinterpret_cast<uint4*>(a.y + (size_t)m * a.N + (size_t)rb_first * 16 + c * 8) = v;
    }
    return;
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
        uint16_t o[4];
#pragma unroll
        for (int i = 0; i < 4; i++) o[i] = float_to_storage(acc[rr][mt][i]);
        *reinterpret_cast<uint2*>(a.y + (size_t)m * a.N + (size_t)rb * 16 + 4 * q) =
            make_uint2((uint32_t)o[0] | ((uint32_t)o[1] << 16), (uint32_t)o[2] | ((uint32_t)o[3] << 16));
      }
    }
  }
}

template <int BITS, int GROUP, bool ZP, int RBW, int MT>
__global__ void __launch_bounds__(256, prefill_min_waves(RBW, MT))
prefill_kernel(const GemmArgs a, int n_tiles, int m_tiles) {
  __shared__ __align__(16) _Float16 lds[prefill_lds_halves(RBW, MT)];
  // Tile order.  Workgroup ids go round-robin over the 8 XCDs, each with its own L2.  The
  // staged tiles remap the ids so that the workgroups of one XCD (ids congruent modulo 8) walk
  // consecutive activation tiles of the same weight rows; the ring tile measured 2-4 % faster
  // in the plain order (every 8th activation tile of all weight tiles on one XCD: two
  // activation tiles, 4 MB, stay in its L2).
  const int total = n_tiles * m_tiles;
  int lid = blockIdx.x;
  if (!prefill_lean(RBW, MT) && (total & 7) == 0) lid = (blockIdx.x & 7) * (total >> 3) + (blockIdx.x >> 3);
  prefill_body<BITS, GROUP, ZP, RBW, MT>(a, lid, m_tiles, 0, lds);
}

// A ring tile with K split over two groups of four waves (see prefill_body): one workgroup per
// CU holds the eight waves that two workgroups of the plain kernel would bring.
template <int BITS, int GROUP, bool ZP, int RBW, int MT>
__global__ void __launch_bounds__(512, 2)
prefill_split_kernel(const GemmArgs a, int m_tiles) {
  __shared__ __align__(16) _Float16 lds[2 * prefill_lds_halves(RBW, MT)];
  prefill_body<BITS, GROUP, ZP, RBW, MT, 2>(a, blockIdx.x, m_tiles, 0, lds);
}

// 128 x 256 tiles with a tail of 128 x 128 tiles.  The larger tile keeps 512 workgroups
// resident (two per CU); when a layer gives it a whole number of such rounds plus a fraction,
// that fraction would run as one more round at the full length of a tile.  Here the first
// `n_big` workgroups take the 128 x 256 tiles of the weight rows below row block `rb_tail`, and
// the rest of the rows go to workgroups with tiles of half the width, which come last, spread
// over twice as many CUs and finish in about half the time.
// (RBW_TAIL 3: the remaining rows as 128 x 192 tiles, where those make up one round of their own and
// 128 x 128 tiles would not fit one)
template <int BITS, int GROUP, bool ZP, int RBW_TAIL = 2>
__global__ void __launch_bounds__(256, 2)
prefill_tail_kernel(const GemmArgs a, int m_tiles, int n_big, int rb_tail) {
  static_assert(prefill_lds_halves(4, 8) == prefill_lds_halves(RBW_TAIL, 8), "both tiles share one LDS block");
  __shared__ __align__(16) _Float16 lds[prefill_lds_halves(4, 8)];
  if ((int)blockIdx.x < n_big)
    prefill_body<BITS, GROUP, ZP, 4, 8>(a, blockIdx.x, m_tiles, 0, lds);
  else
    prefill_body<BITS, GROUP, ZP, RBW_TAIL, 8>(a, blockIdx.x - n_big, m_tiles, rb_tail, lds);
}

// The same split of the weight rows in workgroups of eight waves: the 128 x 256 tiles two to a
// workgroup (PAIR), and the 128 x 128 tiles of the remaining rows one to a workgroup whose two
// groups of four waves take one half of K each.  The narrow tiles then number at most the CUs and
// still run two waves per SIMD, where the kernel above leaves them one.
template <int BITS, int GROUP, bool ZP>
__global__ void __launch_bounds__(512, 2)
prefill_tail8_kernel(const GemmArgs a, int m_tiles, int n_big, int rb_tail) {
  __shared__ __align__(16) _Float16 lds[2 * prefill_lds_halves(4, 8)];
  const int n_pairs = (n_big + 1) / 2;
  if ((int)blockIdx.x < n_pairs)
    prefill_body<BITS, GROUP, ZP, 4, 8, 1, true>(a, blockIdx.x, m_tiles, 0, lds, n_big);
  else
    prefill_body<BITS, GROUP, ZP, 2, 8, 2>(a, blockIdx.x - n_pairs, m_tiles, rb_tail, lds);
}

// Two tile widths sized to fill the resident slots in one round (prefill_mix_wide_tiles): the first
// `n_big` workgroups take 128 x 192 tiles of the weight rows below row block `rb_tail`, the others
// 128 x 128 tiles of the rest.  Workgroups are placed in the order of their ids, the least loaded CU
// first, so a CU ends up with one of each.
template <int BITS, int GROUP, bool ZP>
__global__ void __launch_bounds__(256, 2)
prefill_mix_kernel(const GemmArgs a, int m_tiles, int n_big, int rb_tail) {
  static_assert(prefill_lds_halves(3, 8) == prefill_lds_halves(2, 8), "both tiles share one LDS block");
  __shared__ __align__(16) _Float16 lds[prefill_lds_halves(3, 8)];
  if ((int)blockIdx.x < n_big)
    prefill_body<BITS, GROUP, ZP, 3, 8>(a, blockIdx.x, m_tiles, 0, lds);
  else
    prefill_body<BITS, GROUP, ZP, 2, 8>(a, blockIdx.x - n_big, m_tiles, rb_tail, lds);
}

template <int GROUP, bool ZP>
hipError_t launch_mix(const GemmArgs& a, hipStream_t stream) {
  const int m_tiles = (a.M + 127) / 128;
  int narrow = 0;
  const int wide = prefill_mix_wide_tiles(a.row_blocks, m_tiles, &narrow);
  // (forced on a shape the mix does not apply to: narrow tiles only)
  const int rb_tail = wide * 12;
  const int n_small = wide > 0 ? narrow : (a.row_blocks + 7) / 8;
  const dim3 grid((wide + n_small) * m_tiles), block(256);
  hipLaunchKernelGGL((prefill_mix_kernel<kBits, GROUP, ZP>), grid, block, 0, stream, a, m_tiles, wide * m_tiles, rb_tail);
  return hipGetLastError();
}

template <int GROUP, bool ZP>
hipError_t launch_tail8(const GemmArgs& a, hipStream_t stream) {
  const int m_tiles = (a.M + 127) / 128;
  const int nb = prefill_tail_big_tiles(a.row_blocks, m_tiles);
  const int rb_tail = nb * 16;
  const int n_small = (a.row_blocks - rb_tail + 7) / 8;
  const int n_big = nb * m_tiles;
  const dim3 grid((n_big + 1) / 2 + n_small * m_tiles), block(512);
  hipLaunchKernelGGL((prefill_tail8_kernel<kBits, GROUP, ZP>), grid, block, 0, stream, a, m_tiles, n_big, rb_tail);
  return hipGetLastError();
}

template <int GROUP, bool ZP, int RBW_TAIL = 2>
hipError_t launch_tail(const GemmArgs& a, hipStream_t stream) {
  const int m_tiles = (a.M + 127) / 128;
  const int nb = prefill_tail_big_tiles(a.row_blocks, m_tiles);
  const int rb_tail = nb * 16;
  const int n_small = (a.row_blocks - rb_tail + 4 * RBW_TAIL - 1) / (4 * RBW_TAIL);
  const dim3 grid((nb + n_small) * m_tiles), block(256);
  hipLaunchKernelGGL((prefill_tail_kernel<kBits, GROUP, ZP, RBW_TAIL>), grid, block, 0, stream, a, m_tiles,
                     nb * m_tiles, rb_tail);
  return hipGetLastError();
}

// 128 x 256 and 128 x 192 tiles in one round of all slots (prefill_mix_widest_tiles): the kernel of the
// 192-row tail, with the wide tiles counted by the mix instead of by whole rounds
template <int GROUP, bool ZP>
hipError_t launch_mix_widest(const GemmArgs& a, hipStream_t stream) {
  const int m_tiles = (a.M + 127) / 128;
  int narrow = 0;
  const int wide = prefill_mix_widest_tiles(a.row_blocks, m_tiles, &narrow);
  // (forced on a shape the mix does not apply to: 128 x 192 tiles only)
  const int rb_tail = wide * 16;
  const int n_small = wide > 0 ? narrow : (a.row_blocks + 11) / 12;
  const dim3 grid((wide + n_small) * m_tiles), block(256);
  hipLaunchKernelGGL((prefill_tail_kernel<kBits, GROUP, ZP, 3>), grid, block, 0, stream, a, m_tiles,
                     wide * m_tiles, rb_tail);
  return hipGetLastError();
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

template <int GROUP, bool ZP, int RBW, int MT>
hipError_t launch_split(const GemmArgs& a, hipStream_t stream) {
  const int n_tiles = (a.row_blocks + 4 * RBW - 1) / (4 * RBW);
  const int m_tiles = (a.M + 16 * MT - 1) / (16 * MT);
  const dim3 grid(n_tiles * m_tiles), block(512);
  hipLaunchKernelGGL((prefill_split_kernel<kBits, GROUP, ZP, RBW, MT>), grid, block, 0, stream, a, m_tiles);
  return hipGetLastError();
}

template <int GROUP, bool ZP>
hipError_t launch_shape(const GemmArgs& a, int cfg, hipStream_t s) {
#ifdef MATGPTQ_EXPERIMENT  // one instantiation only: quick compiles while tuning the ring loop
  if constexpr (GROUP == 128 && ZP) return launch_cfg<GROUP, ZP, 4, 8>(a, s);
  else return hipErrorInvalidValue;
#else
  switch (cfg) {
    case 10: return launch_split<GROUP, ZP, 2, 8>(a, s);  // 128 x 128, K split in the workgroup
    case 11: return launch_split<GROUP, ZP, 4, 8>(a, s);  // 128 x 256, K split in the workgroup
    case 0: return launch_cfg<GROUP, ZP, 4, 8>(a, s);   // 128 x 256
    case 1: return launch_cfg<GROUP, ZP, 8, 8>(a, s);   // 128 x 512
    case 2: return launch_cfg<GROUP, ZP, 4, 4>(a, s);   // 64 x 256
    case 3: return launch_cfg<GROUP, ZP, 2, 8>(a, s);   // 128 x 128
    case 4: return launch_cfg<GROUP, ZP, 2, 2>(a, s);   // 32 x 128
    case 5: return launch_cfg<GROUP, ZP, 8, 4>(a, s);   // 64 x 512
    case 6: return launch_cfg<GROUP, ZP, 8, 2>(a, s);   // 32 x 512
    case 8: return launch_tail<GROUP, ZP>(a, s);        // 128 x 256, then a tail of 128 x 128
    case 9: return launch_cfg<GROUP, ZP, 3, 8>(a, s);   // 128 x 192
    case 12: return launch_tail8<GROUP, ZP>(a, s);      // 128 x 256 in pairs, then a tail of 128 x 128 with K split
    case 13: return launch_split<GROUP, ZP, 3, 8>(a, s);  // 128 x 192, K split in the workgroup
    case 14: return launch_mix<GROUP, ZP>(a, s);          // 128 x 192 and 128 x 128, one round of all slots
    case 15: return launch_tail<GROUP, ZP, 3>(a, s);      // 128 x 256, then a tail of 128 x 192
    case 16: return launch_split<GROUP, ZP, 2, 4>(a, s);  // 64 x 128, K split in the workgroup
    case 17: return launch_mix_widest<GROUP, ZP>(a, s);   // 128 x 256 and 128 x 192, one round of all slots
    default: return launch_cfg<GROUP, ZP, 4, 2>(a, s);  // 32 x 256
  }
#endif
}

}  // namespace

#define MATGPTQ_CAT2(a, b) a##b
#define MATGPTQ_CAT(a, b) MATGPTQ_CAT2(a, b)
// cfg selects the workgroup tile (see launch_shape).
#if MATGPTQ_BF16
#define MATGPTQ_LAUNCH_NAME MATGPTQ_CAT(MATGPTQ_CAT(launch_prefill_b, MATGPTQ_BITS), _bf16)
#else
#define MATGPTQ_LAUNCH_NAME MATGPTQ_CAT(launch_prefill_b, MATGPTQ_BITS)
#endif
hipError_t MATGPTQ_LAUNCH_NAME(const GemmArgs& a, int group_size, int cfg,
                                                       hipStream_t stream) {
  const bool zp = a.zeros != nullptr;
  if (group_size == 128)
    return zp ? launch_shape<128, true>(a, cfg, stream) : launch_shape<128, false>(a, cfg, stream);
  if (group_size == 32)
    return zp ? launch_shape<32, true>(a, cfg, stream) : launch_shape<32, false>(a, cfg, stream);
  return zp ? launch_shape<-1, true>(a, cfg, stream) : launch_shape<-1, false>(a, cfg, stream);
}

}  // namespace matgptq
