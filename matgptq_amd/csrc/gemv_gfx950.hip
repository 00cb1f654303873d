// Batch-1..4 kernel: the HBM-bound end of the decode regime (group sizes 128, 32 and -1).
// Compiled once per bitwidth with -DMATGPTQ_BITS=b.
// Role of the reference's gptq_matryoshka_simt
// (inference_lib/matgptq_cuda/csrc/matgptq_gemm.cu:636-953); the design is its own.
//
// Work split.  A workgroup of W waves owns R row blocks (16 weight rows each) and all of
// K.  Wave w owns the tiles [(round W + w) T, +T) of those row blocks, round = 0, 1, ...:
// T consecutive 128-column tiles, i.e. T contiguous KiB-sized pieces of every row block.
// A wave requests everything a round needs at once - the activations of its columns, the
// scales and zeros of its groups, then all R T tiles of codes - and consumes the tiles in
// request order, so the whole round is in flight while the first tile is multiplied.  The
// footprint per wave is small (R T b registers of codes) and many waves are resident.
//
// Arithmetic.  The vector ALU only masks codes into "raw" fp16 pairs 1024 + c 2^p; the
// products run on the matrix cores with the ACTIVATIONS as the 16-row operand and the 16
// weight rows as the 16 columns:  D[i][n] = sum_k A[i][k] raw[n][k].  Row 4u + v of A holds
// batch row v (scaled by 2^-p, as X') during tile u of a group of four tiles and zeros
// otherwise, so that one chain of sixteen MFMAs leaves the sums of four tiles side by side:
// lane (n, q) ends with  sum_k raw X'  of tile q, weight row n, batch rows 0..3 in its four
// accumulator registers.  The same lane holds the scale and zero of exactly that tile and
// row (one 2-byte load per lane fetches the scales of four tiles x 16 rows) and the two
// row-independent sums of that tile,  off = 1024 sum X'  and  xs = sum X, which the wave
// forms while it stages X' (dot products plus a rotate-reduce over the 16 lanes of a tile):
//     acc += scale * (D - off - zero / 2^(8-b) * xs)
// which is  sum_k scale ((c << (8-b)) - zero) x / 2^(8-b)  over the group.  The partial sums
// of the four lane quarters and the W waves meet in LDS once, at the end.
//
// Group size -1 (one scale per weight row) runs the same chain with the one scale in place of
// the tile's.  Group size 32 has a scale per octet of a tile, so there the four ROW GROUPS of A
// take turns per OCTET (row 4j + v is live during the MFMA of octet j): the four MFMAs of one
// tile leave its four octet sums side by side, lane (n, q) holds the scale and zero of octet q
// (again one 2-byte load per lane, now per tile), and the per-octet sums  off  and  xs  travel
// through a small table in LDS (a rotate-reduce over the 4 lanes of an octet fills it).
#include <atomic>

#include "tile_format.h"

#ifndef MATGPTQ_BITS
#error "compile with -DMATGPTQ_BITS={2,3,4,6,8}"
#endif

namespace matgptq {

namespace {

constexpr int kBits = MATGPTQ_BITS;

constexpr int kPreNone = 0, kPreSiluMul = 1, kPreAddRmsNorm = 2;
struct PrologueArgs {
  const uint16_t* b;  // add + norm: the tensor added to the residual stream [M, K], or null
  const uint16_t* w;  // add + norm: the norm's weight [K]
  uint16_t* out;      // add + norm: where the new residual stream goes [M, K], or null
  float eps;
};

__device__ __forceinline__ float dot2(half2v a, half2v b, float c) {
  return __builtin_amdgcn_fdot2(a, b, c, false);
}

// v + (v rotated right by N lanes inside each row of 16 lanes)
template <int N>
__device__ __forceinline__ float add_row_ror(float v) {
  const int r = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x120 + N, 0xF, 0xF, false);
  return v + __int_as_float(r);
}
__device__ __forceinline__ float row_sum16(float v) {
  v = add_row_ror<8>(v);
  v = add_row_ror<4>(v);
  v = add_row_ror<2>(v);
  return add_row_ror<1>(v);
}

// v + the other three lanes of its quad
__device__ __forceinline__ float quad_sum(float v) {
  int r = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, false);  // quad_perm [1,0,3,2]
  v += __int_as_float(r);
  r = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, false);      // quad_perm [2,3,0,1]
  return v + __int_as_float(r);
}

// LDS bytes per wave: X' of one round for MB batch rows + a block of zeros (group 32: as long as
// one batch row's X', so that tile offsets apply to it too) + group 32's table of octet sums
constexpr int gemv_zero_bytes(int t, int group) { return group == 32 ? t * 256 : 256; }
// bytes from one batch row's X' to the next: the four live lanes of an operand read take the
// same 16 bytes of four different batch rows, which a stride of whole KiB would put into the
// same banks
constexpr int gemv_row_bytes(int t, int mb) { return t * 256 + (mb > 1 ? 16 : 0); }
// (eight batch rows: a table of the two sums per batch row and tile)
constexpr int gemv_wave_lds(int t, int mb, int group) {
  return mb * gemv_row_bytes(t, mb) + gemv_zero_bytes(t, group) + (group == 32 ? mb * t * 32 : mb > 4 ? mb * t * 8 : 0);
}
// accumulators per lane and row block: the batch rows of one lane quarter
constexpr int gemv_lane_rows(int mb) { return mb < 4 ? mb : 4; }

// MASTER: `a.packed` holds master-resident bit planes (master_layout.h); the rounded slice to
// BITS is formed in registers while the raw pairs are built.
// PRE: the operator in front of the product is formed while the activations are staged, so that it
// needs no launch and no round trip through memory of its own (group size 128, fp16 storage,
// pre-sliced codes, up to four batch rows):
//   kPreSiluMul     a.x is [M, 2 K]: x = fp16(silu(a.x[:, :K])) * a.x[:, K:], both roundings as two
//                   element-wise operators make them;
//   kPreAddRmsNorm  a.x is the residual stream h [M, K]: v = h + pro.b (one fp16 rounding; pro.b may be
//                   null), x = fp16(v * rsqrt(mean(v^2) + eps) * pro.w), and the first workgroup writes v
//                   to pro.out (another buffer than h: the other workgroups still read h).  The mean
//                   needs every column, so the workgroup's one round must cover all of K.
template <int BITS, bool ZP, int GROUP, int T, int R, int MB, bool MASTER, int PRE = kPreNone>
__device__ __forceinline__ void gemv_body(const GemmArgs& a, const int W, const PrologueArgs& pro) {
  static_assert(PRE == kPreNone || (GROUP == 128 && !MASTER && MB <= 4 && !kBf16), "fused prologues: group 128, pre-sliced, fp16");
  using Fmt = TileFormat<BITS, MASTER>;
  constexpr bool kPerOctet = GROUP == 32;  // a scale per octet: the row groups of A take turns per octet
  static_assert(!kPerOctet || T <= 4, "one lane per 16 bytes of the zero block");
  constexpr int TH = (T + 3) / 4;  // groups of four tiles per round
  // Up to four batch rows the sixteen rows of the activation operand are four tiles x four batch
  // rows and a chain of MFMAs covers four tiles; five to eight batch rows make them two tiles x
  // eight batch rows: a chain covers two tiles, lane (n, q) ends with tile q / 2, batch rows
  // 4 (q % 2) .. + 3, and the sums of a tile travel through a small table in LDS.
  constexpr bool kEight = MB > 4;
  static_assert(!kEight || (!kPerOctet && T % 2 == 0), "eight batch rows: group sizes 128 and -1");
  constexpr int TPC = kEight ? 2 : 4;              // tiles per chain
  constexpr int NC = (T + TPC - 1) / TPC;          // chains per round
  constexpr int NV = gemv_lane_rows(MB);           // accumulators per lane and row block
  constexpr int NS = GROUP == 128 ? NC : GROUP == 32 ? T : 1;  // scale registers per row block
  constexpr float kMul = (float)(1 << (8 - BITS));
  constexpr int kRowBytes = gemv_row_bytes(T, MB);
  constexpr int kXBytes = MB * kRowBytes;
  constexpr int kZeroBytes = gemv_zero_bytes(T, GROUP);
  constexpr int kWaveBytes = gemv_wave_lds(T, MB, GROUP);
  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15;  // weight row inside the row block / row of the activation operand
  const int q = lane >> 4;
  const int rb0 = blockIdx.x * R;

  unsigned char* xw = smem + wave * kWaveBytes;                   // this wave's X' and zeros
  float* red = reinterpret_cast<float*>(smem + W * kWaveBytes);   // [W][R * NV][64]
  float* ssq_part = red + W * R * NV * 64;                        // add + norm: [W][MB] sums of squares
  if (lane * 16 < kZeroBytes) *reinterpret_cast<uint4*>(xw + kXBytes + lane * 16) = make_uint4(0, 0, 0, 0);
  float2* const osum = reinterpret_cast<float2*>(xw + kXBytes + kZeroBytes);  // group 32: [MB][T][4] (off, xs); eight batch rows: [MB][T]

  constexpr uint32_t tile_bytes = Fmt::kTileBytes;
  const typename Fmt::Consts consts;
  // activation operand: row n of A is batch row n % 4 while tile u = n / 4 of a group of four is
  // multiplied; the batch rows beyond M repeat row M - 1 (their results are never stored)
  // (eight batch rows: row n is batch row n % 8 during tile n / 8 of a pair of tiles)
  const int brow = kEight ? (n & 7) : (n & 3);
  const int slot = kEight ? (n >> 3) : (n >> 2);
  const int arow = brow < a.M ? brow : a.M - 1;
  const unsigned char* a_live = xw + (MB > 1 ? arow * kRowBytes : 0) + q * 16;
  const unsigned char* a_zero = xw + kXBytes + q * 16;

  float acc[R][NV];
#pragma unroll
  for (int rr = 0; rr < R; rr++)
#pragma unroll
    for (int v = 0; v < NV; v++) acc[rr][v] = 0.f;

  for (int kt0 = wave * T; kt0 < a.k_tiles; kt0 += W * T) {
    const int left = a.k_tiles - kt0;
    const int nt = left < T ? left : T;  // tiles of this round

    // ---- requests, oldest first: activations, scales and zeros, codes.  Every request is
    // unconditional; what lies past the round is cut off by the size of its descriptor and
    // reads as zero (zero scale: such a tile adds nothing).
    u32x4 xv[MB][TH];
    u32x4 xu[PRE == kPreNone ? 1 : MB][TH];  // second operand of the prologue (up half, or the added tensor)
    u32x4 xn[TH];                            // add + norm: the norm's weights of these columns
#pragma unroll
    for (int m = 0; m < MB; m++) {
      const int mrow = m < a.M ? m : a.M - 1;
      const size_t row = (size_t)mrow * (PRE == kPreSiluMul ? 2 * (size_t)a.K : (size_t)a.K);
      const BufRsrc xr = make_rsrc(a.x + row, (uint32_t)(kt0 + nt) * 256u);
#pragma unroll
      for (int h = 0; h < TH; h++)
        xv[m][h] = __builtin_amdgcn_raw_buffer_load_b128(xr, lane * 16, (uint32_t)(kt0 + 4 * h) * 256u, 0);
      if constexpr (PRE != kPreNone) {
        const uint16_t* second = PRE == kPreSiluMul ? a.x + row + a.K : pro.b != nullptr ? pro.b + row : a.x;
        const BufRsrc ur = make_rsrc(second, PRE == kPreAddRmsNorm && pro.b == nullptr ? 0u : (uint32_t)(kt0 + nt) * 256u);
#pragma unroll
        for (int h = 0; h < TH; h++)
          xu[m][h] = __builtin_amdgcn_raw_buffer_load_b128(ur, lane * 16, (uint32_t)(kt0 + 4 * h) * 256u, 0);
      }
    }
    if constexpr (PRE == kPreAddRmsNorm) {
      const BufRsrc nr = make_rsrc(pro.w, (uint32_t)(kt0 + nt) * 256u);
#pragma unroll
      for (int h = 0; h < TH; h++)
        xn[h] = __builtin_amdgcn_raw_buffer_load_b128(nr, lane * 16, (uint32_t)(kt0 + 4 * h) * 256u, 0);
    }
    uint16_t sv[R][NS], zv[R][NS];
    uint32_t w[R][T][Fmt::kWords];
#pragma unroll
    for (int rr = 0; rr < R; rr++) {
      const bool rows = rb0 + rr < a.row_blocks;
      const uint32_t g0 = (uint32_t)(rb0 + rr) * a.k_tiles + kt0;  // first tile of the round
      // scales of a row block: G groups of 16 values; a tile spans one group (32 bytes), or four at
      // group size 32 (G may then be 4 K/128 + 2: the last 64 columns are not this kernel's)
      const uint32_t sg0 = (uint32_t)(rb0 + rr) * a.G + (GROUP == 32 ? 4u : 1u) * kt0;  // first group of the round
      constexpr uint32_t kSB = GROUP == 128 ? 32u : 128u;
      const uint32_t s_end = GROUP == -1 ? (uint32_t)(rb0 + rr + 1) * 32u : sg0 * 32u + nt * kSB;
      const BufRsrc sr = make_rsrc(a.scales, rows ? s_end : 0u);
      const BufRsrc zr = make_rsrc(ZP ? a.zeros : a.scales, rows ? s_end : 0u);
#pragma unroll
      for (int h = 0; h < NS; h++) {
        // lane (n, q): group 128, the scale of row n in tile 4 h + q (eight batch rows: 2 h + q / 2);
        // group 32, in octet q of tile h
        const uint32_t lo = GROUP == -1 ? (uint32_t)n * 2u : kEight ? (uint32_t)((q >> 1) * 16 + n) * 2u : (uint32_t)lane * 2u;
        const uint32_t so = GROUP == -1 ? (uint32_t)(rb0 + rr) * 32u : (sg0 + TPC * h) * 32u;  // (group 32: h = tile)
        sv[rr][h] = __builtin_amdgcn_raw_buffer_load_b16(sr, lo, so, 0);
        if constexpr (ZP) zv[rr][h] = __builtin_amdgcn_raw_buffer_load_b16(zr, lo, so, 0);
      }
    }
#pragma unroll
    for (int rr = 0; rr < R; rr++) {
      const bool rows = rb0 + rr < a.row_blocks;
      const uint32_t g0 = (uint32_t)(rb0 + rr) * a.k_tiles + kt0;
      const BufRsrc wr = make_rsrc(a.packed, rows ? (g0 + nt) * tile_bytes : 0u);
#pragma unroll
      for (int i = 0; i < T; i++) Fmt::load(wr, (g0 + i) * tile_bytes, lane, w[rr][i]);
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- stage X' = X 2^-p (lane: chunk lane % 16 of tile 4 h + lane / 16) and form the two
    // sums of every tile; after the rotate-reduce each lane of quarter q holds those of tile 4 h + q
    float off[MB][TH], xs[MB][TH];
    const half2v ones = h2_splat(1.0f);
    if constexpr (PRE == kPreSiluMul) {
#pragma unroll
      for (int m = 0; m < MB; m++)
#pragma unroll
        for (int h = 0; h < TH; h++) {
          Frag g, u;
          g.v = make_uint4(xv[m][h].x, xv[m][h].y, xv[m][h].z, xv[m][h].w);
          u.v = make_uint4(xu[m][h].x, xu[m][h].y, xu[m][h].z, xu[m][h].w);
#pragma unroll
          for (int e = 0; e < 8; e++) {
            const float x = (float)g.h[e];
            g.h[e] = (_Float16)(x / (1.0f + __expf(-x))) * u.h[e];
          }
          xv[m][h] = u32x4{g.u[0], g.u[1], g.u[2], g.u[3]};
        }
    } else if constexpr (PRE == kPreAddRmsNorm) {
      float ssq[MB];
#pragma unroll
      for (int m = 0; m < MB; m++) {
        ssq[m] = 0.f;
#pragma unroll
        for (int h = 0; h < TH; h++) {
          Frag v, d;
          v.v = make_uint4(xv[m][h].x, xv[m][h].y, xv[m][h].z, xv[m][h].w);
          d.v = make_uint4(xu[m][h].x, xu[m][h].y, xu[m][h].z, xu[m][h].w);  // zeros when nothing is added
          v.h = v.h + d.h;
          if (blockIdx.x == 0 && pro.out != nullptr && m < a.M && 4 * h + q < nt)
            *reinterpret_cast<uint4*>(pro.out + (size_t)m * a.K + (size_t)(kt0 + 4 * h) * 128 + lane * 8) = v.v;
#pragma unroll
          for (int i = 0; i < 4; i++) ssq[m] = dot2(v.p[i], v.p[i], ssq[m]);
          xv[m][h] = u32x4{v.u[0], v.u[1], v.u[2], v.u[3]};
        }
        float t = row_sum16(ssq[m]);
        t += __shfl_xor(t, 16);
        t += __shfl_xor(t, 32);
        if (lane == 0) ssq_part[wave * MB + m] = t;
      }
      __syncthreads();  // every wave is here: the one round covers all of K (checked by the launcher)
#pragma unroll
      for (int m = 0; m < MB; m++) {
        float total = 0.f;
        for (int w2 = 0; w2 < W; w2++) total += ssq_part[w2 * MB + m];
        const float rs = rsqrtf(total / (float)a.K + pro.eps);
#pragma unroll
        for (int h = 0; h < TH; h++) {
          Frag v, wn;
          v.v = make_uint4(xv[m][h].x, xv[m][h].y, xv[m][h].z, xv[m][h].w);
          wn.v = make_uint4(xn[h].x, xn[h].y, xn[h].z, xn[h].w);
#pragma unroll
          for (int e = 0; e < 8; e++) v.h[e] = (_Float16)((float)v.h[e] * rs * (float)wn.h[e]);
          xv[m][h] = u32x4{v.u[0], v.u[1], v.u[2], v.u[3]};
        }
      }
    }
#pragma unroll
    for (int m = 0; m < MB; m++) {
#pragma unroll
      for (int h = 0; h < TH; h++) {
        Frag v;
        v.v = make_uint4(xv[m][h].x, xv[m][h].y, xv[m][h].z, xv[m][h].w);
        v.h = storage8_to_half8(v.h);
        float sx = dot2(v.p[0], ones, 0.f);
        sx = dot2(v.p[1], ones, sx);
        sx = dot2(v.p[2], ones, sx);
        sx = dot2(v.p[3], ones, sx);
        if constexpr (Fmt::kScaledX) {
          // pair i of octet j is scaled by 2^-p(j, i); only pre-sliced 2-bit codes depend on j (its parity)
          const bool odd = BITS == 2 && !MASTER && (n & 4) != 0;  // octet = chunk / 4, chunk = lane % 16
          const float i0 = 1.0f / (float)(1 << Fmt::raw_shift(0, 0)), i1 = 1.0f / (float)(1 << Fmt::raw_shift(0, 1));
          const float i2 = 1.0f / (float)(1 << Fmt::raw_shift(0, 2)), i3 = 1.0f / (float)(1 << Fmt::raw_shift(0, 3));
          const float o0 = 1.0f / (float)(1 << Fmt::raw_shift(1, 0)), o1 = 1.0f / (float)(1 << Fmt::raw_shift(1, 1));
          const float o2 = 1.0f / (float)(1 << Fmt::raw_shift(1, 2)), o3 = 1.0f / (float)(1 << Fmt::raw_shift(1, 3));
          v.p[0] = v.p[0] * h2_splat(odd ? o0 : i0);
          v.p[1] = v.p[1] * h2_splat(odd ? o1 : i1);
          v.p[2] = v.p[2] * h2_splat(odd ? o2 : i2);
          v.p[3] = v.p[3] * h2_splat(odd ? o3 : i3);
        }
        float so = dot2(v.p[0], ones, 0.f);
        so = dot2(v.p[1], ones, so);
        so = dot2(v.p[2], ones, so);
        so = dot2(v.p[3], ones, so);
        if (T >= 4 || 4 * h + q < T)
          *reinterpret_cast<uint4*>(xw + m * kRowBytes + h * 1024 + lane * 16) = v.v;
        if constexpr (kEight) {
          // the first lane of a quarter files the sums of its tile under (batch row, tile)
          xs[m][h] = row_sum16(sx);
          off[m][h] = 1024.0f * row_sum16(so);
          if (n == 0 && 4 * h + q < T) osum[m * T + 4 * h + q] = make_float2(off[m][h], xs[m][h]);
        } else if constexpr (kPerOctet) {
          // sums over the four chunks of an octet; the first lane of the quad files them under
          // (batch row, tile 4 h + lane / 16, octet chunk / 4)
          const float2 pair = make_float2(1024.0f * quad_sum(so), quad_sum(sx));
          if ((lane & 3) == 0 && (T >= 4 || 4 * h + q < T)) osum[(m * T + 4 * h + q) * 4 + (n >> 2)] = pair;
          xs[m][h] = 0.f;
          off[m][h] = 0.f;
        } else {
          xs[m][h] = row_sum16(sx);
          off[m][h] = 1024.0f * row_sum16(so);
        }
      }
    }

    // ---- the tiles, in request order
    float4v d[R];
#pragma unroll
    for (int rr = 0; rr < R; rr++) d[rr] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < T; i++) {
      const int u = i & (TPC - 1);
      Frag av[4];
      if constexpr (kPerOctet) {
        // octet j: row group j live (the zero block is as long as X', so `i * 256` applies to both)
#pragma unroll
        for (int j = 0; j < 4; j++)
          av[j].v = *reinterpret_cast<const uint4*>(((n >> 2) == j ? a_live : a_zero) + i * 256 + j * 64);
      } else {
        const unsigned char* ab = slot == u ? a_live + i * 256 : a_zero;
#pragma unroll
        for (int j = 0; j < 4; j++) av[j].v = *reinterpret_cast<const uint4*>(ab + j * 64);
      }
#pragma unroll
      for (int rr = 0; rr < R; rr++) {
        Frag bw;
        Fmt::template raw<0>(w[rr][i], consts, bw.u);
        d[rr] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[0].h, bw.h, d[rr], 0, 0, 0);
        Fmt::template raw<1>(w[rr][i], consts, bw.u);
        d[rr] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[1].h, bw.h, d[rr], 0, 0, 0);
        Fmt::template raw<2>(w[rr][i], consts, bw.u);
        d[rr] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[2].h, bw.h, d[rr], 0, 0, 0);
        Fmt::template raw<3>(w[rr][i], consts, bw.u);
        d[rr] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[3].h, bw.h, d[rr], 0, 0, 0);
      }
      if (kPerOctet || u == TPC - 1 || i == T - 1) {
        const int h = i >> 2;
        const int si = GROUP == 128 ? i / TPC : GROUP == 32 ? i : 0;
        float fo[NV], fx[NV];
#pragma unroll
        for (int v = 0; v < NV; v++) {
          if constexpr (kEight) {
            const float2 pair = osum[((q & 1) * 4 + v) * T + (i / TPC) * TPC + (q >> 1)];
            fo[v] = pair.x;
            fx[v] = pair.y;
          } else if constexpr (kPerOctet) {
            const float2 pair = osum[(v * T + i) * 4 + q];
            fo[v] = pair.x;
            fx[v] = pair.y;
          } else {
            fo[v] = off[v][h];
            fx[v] = xs[v][h];
          }
        }
#pragma unroll
        for (int rr = 0; rr < R; rr++) {
          const float s = storage_to_float(sv[rr][si]);
          float zs = (float)(1 << (BITS - 1));
          if constexpr (ZP) zs = storage_to_float(zv[rr][si]) * (1.0f / kMul);
#pragma unroll
          for (int v = 0; v < NV; v++) acc[rr][v] += s * (d[rr][v] - fo[v] - zs * fx[v]);
          d[rr] = float4v{0.f, 0.f, 0.f, 0.f};
        }
      }
    }
  }

  // ---- the lane quarters that hold the same batch rows and the W waves meet: red[wave][rr * NV + v][lane]
#pragma unroll
  for (int rr = 0; rr < R; rr++)
#pragma unroll
    for (int v = 0; v < NV; v++) red[((wave * R + rr) * NV + v) * 64 + lane] = acc[rr][v];
  __syncthreads();
  for (int o = wave; o < R * NV; o += W) {
    float sum = 0.f;
    for (int w2 = 0; w2 < W; w2++) sum += red[(w2 * R * NV + o) * 64 + lane];
    if constexpr (!kEight) sum += __shfl_xor(sum, 16);
    sum += __shfl_xor(sum, 32);
    const int rr = o / NV;
    const int v = o - rr * NV + (kEight ? q * 4 : 0);  // batch row (eight: quarters 0 and 1 hold rows 0..3 and 4..7)
    if (q < (kEight ? 2 : 1) && rb0 + rr < a.row_blocks && v < a.M)
      a.y[(size_t)v * a.N + (size_t)(rb0 + rr) * 16 + n] = float_to_storage(sum * kMul);
  }
}

// WPE: waves per SIMD the register allocation is held to
template <int BITS, bool ZP, int GROUP, int T, int R, int MB, int WPE, bool MASTER, int PRE = kPreNone>
__global__ void __launch_bounds__(1024, WPE) gemv_kernel(const GemmArgs a, const int W, const PrologueArgs pro) {
  gemv_body<BITS, ZP, GROUP, T, R, MB, MASTER, PRE>(a, W, pro);
}

template <bool ZP, int GROUP, int T, int R, int MB, int WPE, bool MASTER, int PRE = kPreNone>
hipError_t launch_one(const GemmArgs& a, int W, size_t lds_pad, hipStream_t stream, const PrologueArgs& pro = PrologueArgs{}) {
  const dim3 grid((a.row_blocks + R - 1) / R), block(64 * W);
  size_t smem = (size_t)W * gemv_wave_lds(T, MB, GROUP) + (size_t)W * R * gemv_lane_rows(MB) * 256 +
                (PRE == kPreAddRmsNorm ? (size_t)W * MB * 4 : 0);
  // add + norm: the workgroup's one round has to cover all of K, with every wave taking part
  if (PRE == kPreAddRmsNorm && (W * T < a.k_tiles || (W - 1) * T >= a.k_tiles)) return hipErrorInvalidValue;
  if (smem < lds_pad) smem = lds_pad;
  if (W < 1 || W > 16 || a.M > MB || smem > 160 * 1024) return hipErrorInvalidValue;
  if (smem > 64 * 1024) {
    // more than 64 KiB of dynamic LDS has to be allowed once per kernel and device (the attribute
    // belongs to the device's copy of the code object): one bit per device, set after the call succeeded
    static std::atomic<uint64_t> allowed{0};
    int dev = 0;
    if (const hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
    const uint64_t bit = 1ull << (dev & 63);
    if (dev >= 64 || !(allowed.load(std::memory_order_acquire) & bit)) {
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemv_kernel<kBits, ZP, GROUP, T, R, MB, WPE, MASTER, PRE>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
      if (e != hipSuccess) return e;
      if (dev < 64) allowed.fetch_or(bit, std::memory_order_release);
    }
  }
  hipLaunchKernelGGL((gemv_kernel<kBits, ZP, GROUP, T, R, MB, WPE, MASTER, PRE>), grid, block, smem, stream, a, W, pro);
  return hipGetLastError();
}

// the fused prologues: shapes (4, 1) and (4, 2), one, two or up to four batch rows
template <bool ZP, int PRE>
hipError_t launch_prologue(const GemmArgs& a, int shape, int W, const PrologueArgs& pro, hipStream_t s) {
  if constexpr (kBf16) {
    return hipErrorInvalidValue;
  } else {
    if (shape != 1 && shape != 2) return hipErrorInvalidValue;
#define MATGPTQ_PRE_CASE(MBV)                                                                    \
    return shape == 1 ? launch_one<ZP, 128, 4, 1, MBV, 4, false, PRE>(a, W, 0, s, pro)          \
                      : launch_one<ZP, 128, 4, 2, MBV, 4, false, PRE>(a, W, 0, s, pro);
    if (a.M == 1) { MATGPTQ_PRE_CASE(1) }
    if (a.M == 2) { MATGPTQ_PRE_CASE(2) }
    if (a.M <= 4) { MATGPTQ_PRE_CASE(4) }
#undef MATGPTQ_PRE_CASE
    return hipErrorInvalidValue;
  }
}

// shapes built: (T tiles per wave and round, R row blocks per workgroup); the master-resident
// storage and the group sizes 32 and -1 take the two shapes the planner uses
template <bool ZP, int GROUP, int MB, bool MASTER>
hipError_t launch_shape(const GemmArgs& a, int shape, int W, size_t lds_pad, hipStream_t s) {
  if constexpr (MASTER || GROUP != 128 || MB > 4) {
    if (shape == 2) return launch_one<ZP, GROUP, 4, 2, MB, 4, MASTER>(a, W, lds_pad, s);
    if (shape == 1) return launch_one<ZP, GROUP, 4, 1, MB, 4, MASTER>(a, W, lds_pad, s);
    return hipErrorInvalidValue;
  } else {
    switch (shape) {
      case 0: return launch_one<ZP, 128, 8, 1, MB, 4, false>(a, W, lds_pad, s);
      case 1: return launch_one<ZP, 128, 4, 1, MB, 4, false>(a, W, lds_pad, s);
      case 2: return launch_one<ZP, 128, 4, 2, MB, 4, false>(a, W, lds_pad, s);
      case 3: return launch_one<ZP, 128, 2, 2, MB, 4, false>(a, W, lds_pad, s);
      case 4: return launch_one<ZP, 128, 2, 4, MB, 4, false>(a, W, lds_pad, s);
      case 6: return launch_one<ZP, 128, 4, 4, MB, 4, false>(a, W, lds_pad, s);
      default: return launch_one<ZP, 128, 2, 1, MB, 4, false>(a, W, lds_pad, s);
    }
  }
}

template <int GROUP, bool MASTER>
hipError_t launch_storage(const GemmArgs& a, int shape, int W, size_t lds_pad, hipStream_t stream) {
  const bool zp = a.zeros != nullptr;
  if (a.M == 1)
    return zp ? launch_shape<true, GROUP, 1, MASTER>(a, shape, W, lds_pad, stream)
              : launch_shape<false, GROUP, 1, MASTER>(a, shape, W, lds_pad, stream);
  if (a.M == 2)
    return zp ? launch_shape<true, GROUP, 2, MASTER>(a, shape, W, lds_pad, stream)
              : launch_shape<false, GROUP, 2, MASTER>(a, shape, W, lds_pad, stream);
  if (a.M <= 4)
    return zp ? launch_shape<true, GROUP, 4, MASTER>(a, shape, W, lds_pad, stream)
              : launch_shape<false, GROUP, 4, MASTER>(a, shape, W, lds_pad, stream);
  // five to eight batch rows: one scale per tile or row
  if constexpr (GROUP != 32)
    return zp ? launch_shape<true, GROUP, 8, MASTER>(a, shape, W, lds_pad, stream)
              : launch_shape<false, GROUP, 8, MASTER>(a, shape, W, lds_pad, stream);
  return hipErrorInvalidValue;
}

}  // namespace

// Entry of this translation unit.  shape: index into the (T, R) table above; W: waves per
// workgroup (1..16); lds_pad: dynamic LDS to ask for when it exceeds what the kernel needs
// (limits how many workgroups share a CU); master: `a.packed` holds master-resident bit planes
// (shapes 1 and 2); group sizes 32 and -1: shapes 1 and 2.  M <= 4; five to eight batch rows with
// group size 128 or -1, shapes 1 and 2.
#define MATGPTQ_CAT2(a, b) a##b
#define MATGPTQ_CAT(a, b) MATGPTQ_CAT2(a, b)
#if MATGPTQ_BF16
#define MATGPTQ_LAUNCH_NAME MATGPTQ_CAT(MATGPTQ_CAT(launch_gemv_b, MATGPTQ_BITS), _bf16)
#else
#define MATGPTQ_LAUNCH_NAME MATGPTQ_CAT(launch_gemv_b, MATGPTQ_BITS)
#endif
#if MATGPTQ_BF16
#define MATGPTQ_PRE_LAUNCH_NAME MATGPTQ_CAT(MATGPTQ_CAT(launch_gemv_prologue_b, MATGPTQ_BITS), _bf16)
#else
#define MATGPTQ_PRE_LAUNCH_NAME MATGPTQ_CAT(launch_gemv_prologue_b, MATGPTQ_BITS)
#endif
// The gemv kernel with a fused prologue (kind 1: SiLU gate, 2: residual add + RMS norm); group size
// 128, fp16 storage, up to four batch rows, shapes 1 and 2.
hipError_t MATGPTQ_PRE_LAUNCH_NAME(const GemmArgs& a, int kind, int shape, int W, const void* b, const void* w,
                                   void* out, float eps, hipStream_t stream) {
  const PrologueArgs pro{static_cast<const uint16_t*>(b), static_cast<const uint16_t*>(w), static_cast<uint16_t*>(out), eps};
  const bool zp = a.zeros != nullptr;
  if (kind == kPreSiluMul)
    return zp ? launch_prologue<true, kPreSiluMul>(a, shape, W, pro, stream)
              : launch_prologue<false, kPreSiluMul>(a, shape, W, pro, stream);
  if (kind == kPreAddRmsNorm)
    return zp ? launch_prologue<true, kPreAddRmsNorm>(a, shape, W, pro, stream)
              : launch_prologue<false, kPreAddRmsNorm>(a, shape, W, pro, stream);
  return hipErrorInvalidValue;
}

hipError_t MATGPTQ_LAUNCH_NAME(const GemmArgs& a, int group_size, int shape, int W, size_t lds_pad, bool master,
                               hipStream_t stream) {
  if (group_size == 32)
    return master ? launch_storage<32, true>(a, shape, W, lds_pad, stream)
                  : launch_storage<32, false>(a, shape, W, lds_pad, stream);
  if (group_size == -1)
    return master ? launch_storage<-1, true>(a, shape, W, lds_pad, stream)
                  : launch_storage<-1, false>(a, shape, W, lds_pad, stream);
  return master ? launch_storage<128, true>(a, shape, W, lds_pad, stream)
                : launch_storage<128, false>(a, shape, W, lds_pad, stream);
}

}  // namespace matgptq
