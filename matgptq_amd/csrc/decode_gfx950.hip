// Decode-regime kernel (M <= 16): HBM-bound product of packed b-bit codes with a
// few activation rows.  Compiled once per bitwidth with -DMATGPTQ_BITS=b.
// Role of the reference's gptq_matryoshka_simt / gptq_matryoshka at small batch
// (inference_lib/matgptq_cuda/csrc/matgptq_gemm.cu:337-953); the design is its own.
//
// Work split.  A workgroup has S*W waves and owns S*R row blocks (16 rows each)
// and all of K.  Wave (s, w) owns the R row blocks of slot s and the 128-column
// tiles w, w+W, ... of those rows; it streams them with one coalesced 16-byte
// load per lane and segment, U tiles per pipeline stage.  Two flavours:
//   stream : the next stage is in flight while the current one is consumed
//            (two register buffers, fewer waves per SIMD) - long tile runs;
//   burst  : one register buffer, more waves per SIMD - short tile runs.
// The W partial sums of a slot meet in LDS at the end.
//
// Arithmetic.  The VALU only masks the codes into "raw" fp16 pairs
// 1024 + c*2^p (one v_and_or_b32 / v_perm_b32 per two codes).  Everything else
// runs on the matrix cores, with fp32 accumulation, on X' = X * 2^-p staged in LDS
// (p depends only on the position inside an octet; once per workgroup for M > 1, while at
// M = 1 every wave stages just the columns of its own tiles and starts without a barrier):
//     D += raw        * X'      ->  sum (1024*2^-p + c) x
//     D -= (1024 + 2^(b-1) 2^p) * X'   (constant operand)  ->  sum (c - 2^(b-1)) x
//     D -= (zero-128)/2^(8-b) 2^p * X' (one value per row and group, zero-point form only)
// so D = sum_k ((c << (8-b)) - zero) x / 2^(8-b) over the group, exact products.
// Per group the fp32 D is multiplied by the group scale in fp32 and added to
// the running sum; 2^(8-b) is applied to the final value.  The constant-operand chain
// does not depend on the row, so it is computed once per tile and the chains of the R
// row blocks of a wave start from it.
#include "device_common.h"

#ifndef MATGPTQ_BITS
#error "compile with -DMATGPTQ_BITS={2,3,4,6,8}"
#endif

namespace matgptq {

namespace {

constexpr int kBits = MATGPTQ_BITS;

// Tiles a wave loads per pipeline stage, for R row blocks per wave.
// Group 32 carries four scales (and zeros) per tile and row block, so fewer tiles fit.
constexpr int tiles_in_flight(int bits, int r, int group = 128) {
  const int u = (16 + r * bits - 1) / (r * bits);
  const int cap = group == 32 ? (r >= 4 ? 1 : 2) : 4;
  return u < 1 ? 1 : (u > cap ? cap : u);
}

// fp16 pair constant for pair i of octet J: 2^p in both halves, times `f`.
template <int BITS, int J, int I>
__device__ __forceinline__ half2v pow_pair(float f) {
  return h2_splat(f * (float)(1 << Codec<BITS>::raw_shift(J, I)));
}

template <int BITS, int J, int I>
__device__ __forceinline__ half2v inv_pow_pair() {
  return h2_splat(1.0f / (float)(1 << Codec<BITS>::raw_shift(J, I)));
}

struct DecodeShape {
  int S, W;     // slots and k-slices per workgroup
  int kc;       // tiles of K whose activations are staged in LDS at a time
  int lg_rows;  // log2(S * R * 16)
};

template <int BITS, int R, int U, int GPT, bool ZP>
struct Stage {
  uint32_t w[U][R][BITS];
  uint2 s[U][R][GPT];              // scales of rows 4q..4q+3 (accumulator layout)
  _Float16 z[ZP ? U : 1][R][GPT];  // zero of row lane%16 (operand layout)
};

// STREAM: double-buffered stages.  CHUNKED: X' is staged kc tiles at a time.
template <int BITS, int GROUP, bool ZP, int R, bool STREAM, bool CHUNKED>
__device__ __forceinline__ void decode_body(const GemmArgs& a, const DecodeShape sh) {
  constexpr int U = tiles_in_flight(BITS, R, GROUP);
  constexpr bool GROUPED = GROUP != -1;
  constexpr int GPT = GROUP == 32 ? 4 : 1;  // groups per tile
  constexpr float kMul = (float)(1 << (8 - BITS));
  extern __shared__ __align__(16) unsigned char smem[];
  const int S = sh.S, W = sh.W, kc = sh.kc;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps tile math scalar
  const int slot = wave / W;
  const int ws = wave - slot * W;
  const int r16 = lane & 15;  // row of the weight operand / batch column of the x operand
  const int q = lane >> 4;
  const int rb_wg = blockIdx.x * S * R;  // first row block of the workgroup
  const int rb0 = rb_wg + slot * R;      // first row block of this wave
  const bool live = rb0 < a.row_blocks;  // the last workgroup may have idle slots

  // LDS: [ partial sums | X' ]
  float* red = reinterpret_cast<float*>(smem);                                  // [S*W][R][256]
  _Float16* xs = reinterpret_cast<_Float16*>(smem + (size_t)S * W * R * 1024);  // [M][kc*128 + 8]
  const int pitch = kc * 128 + 8;
  // Operand columns beyond M are never stored, so those lanes simply re-read row M-1.
  const int xrow = r16 < a.M ? r16 : a.M - 1;
  const _Float16* xb = xs + xrow * pitch + q * 8;

  constexpr uint32_t tile_bytes = (uint32_t)tile_words(BITS) * 4;
  const uint32_t rb_bytes = (uint32_t)a.k_tiles * tile_bytes;
  const uint32_t aux_bytes = (uint32_t)a.row_blocks * a.G * 32;  // scales / zeros: [N/16][G][16] halves
  const uint32_t w_bytes = (uint32_t)a.row_blocks * rb_bytes;

  using StageT = Stage<BITS, R, U, GPT, ZP>;
  StageT cur, nxt;
  const UnpackConsts<BITS> kc_unpack;

  // loads stage `stage` of chunk [c0, c1): tiles c0 + ws + W * (stage * U + u).  Branch-free:
  // a tile beyond the chunk is read through a descriptor of zero length (every lane out of
  // range, nothing fetched), so that the count of loads in flight is known at compile time
  // and later waits can be exact.
  auto load_stage = [&](StageT& st, int c0, int c1, int stage) {
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int t = c0 + ws + W * (stage * U + u);
      const bool valid = live && t < c1;
      const BufRsrc wr = make_rsrc(a.packed, valid ? w_bytes : 0u);
      const BufRsrc sr = make_rsrc(a.scales, valid ? aux_bytes : 0u);
      const BufRsrc zr = make_rsrc(ZP ? a.zeros : a.scales, valid ? aux_bytes : 0u);
#pragma unroll
      for (int rr = 0; rr < R; rr++) {
        load_tile_words<BITS>(wr, (uint32_t)(rb0 + rr) * rb_bytes + (uint32_t)t * tile_bytes, lane,
                              st.w[u][rr]);
        if constexpr (GROUPED) {
#pragma unroll
          for (int gg = 0; gg < GPT; gg++) {
            const uint32_t so = ((uint32_t)(rb0 + rr) * a.G + (uint32_t)t * GPT + gg) * 32;  // bytes
            const u32x2 sv = __builtin_amdgcn_raw_buffer_load_b64(sr, q * 8, so, 0);
            st.s[u][rr][gg] = make_uint2(sv.x, sv.y);
            if constexpr (ZP) {
              const uint16_t zv = __builtin_amdgcn_raw_buffer_load_b16(zr, r16 * 2, so, 0);
              st.z[u][rr][gg] = storage_to_half(zv);
            }
          }
        }
      }
    }
    // all loads of a stage are issued before anything that uses them
    __builtin_amdgcn_sched_barrier(0);
  };

  auto scale_x = [&](half8& hv, bool odd) {
    if constexpr (BITS != 8) {
      Frag v;
      v.h = hv;
      if (odd) {
        v.p[0] = v.p[0] * inv_pow_pair<BITS, 1, 0>();
        v.p[1] = v.p[1] * inv_pow_pair<BITS, 1, 1>();
        v.p[2] = v.p[2] * inv_pow_pair<BITS, 1, 2>();
        v.p[3] = v.p[3] * inv_pow_pair<BITS, 1, 3>();
      } else {
        v.p[0] = v.p[0] * inv_pow_pair<BITS, 0, 0>();
        v.p[1] = v.p[1] * inv_pow_pair<BITS, 0, 1>();
        v.p[2] = v.p[2] * inv_pow_pair<BITS, 0, 2>();
        v.p[3] = v.p[3] * inv_pow_pair<BITS, 0, 3>();
      }
      hv = v.h;
    }
  };
  // The copy of X' is latency-bound: a thread keeps XU loads in flight, and the first trip
  // is issued BEFORE the weight loads of the first stage (memory returns in order, so an
  // activation load queued behind them would not be usable until all of them had landed).
  constexpr int XU = 4;
  struct XTrip {
    half8 v[XU];
    int dst[XU];   // halves into xs
    bool odd[XU];  // b = 2: parity of the octet index k/32 selects the shift set
  };
  auto x_fetch = [&](XTrip& t, int c0, int chunks, int base) {
    const half8* src = reinterpret_cast<const half8*>(a.x + (size_t)c0 * 128);
    const int total = a.M * chunks;
    int off[XU];
#pragma unroll
    for (int i = 0; i < XU; i++) {
      const int idx = base + i * (int)blockDim.x;
      // Past the end a thread repeats the last chunk (same value to the same place): loads and
      // stores stay unconditional, so none of them can be moved behind the weight loads.
      const int cl = idx < total ? idx : total - 1;
      int m = 0, c = cl;
      if (a.M > 1) {
        m = cl / chunks;
        c = cl - m * chunks;
      }
      off[i] = m * (a.K / 8) + c;
      t.dst[i] = m * pitch + c * 8;
      t.odd[i] = BITS == 2 && ((c >> 2) & 1) != 0;  // octet index k/32 = c/4
    }
    // straight-line loads: the compiler can then wait for exactly these and no later load
#pragma unroll
    for (int i = 0; i < XU; i++) t.v[i] = src[off[i]];
  };
  auto x_commit = [&](XTrip& t) {
#pragma unroll
    for (int i = 0; i < XU; i++) {
      t.v[i] = storage8_to_half8(t.v[i]);
      scale_x(t.v[i], t.odd[i]);
      *reinterpret_cast<half8*>(xs + t.dst[i]) = t.v[i];
    }
  };
  // stores the prefetched first trip `t`, then copies the rest of columns [c0*128, c1*128)
  auto stage_x = [&](XTrip& t, int c0, int c1) {
    const int chunks = (c1 - c0) * 16;
    const int total = a.M * chunks;
    const int step = XU * (int)blockDim.x;
    x_commit(t);
    for (int base = tid + step; base < total; base += step) {
      x_fetch(t, c0, chunks, base);
      x_commit(t);
    }
  };

  float4v acc[R];  // sum over groups of scale * D
  float4v d[R];    // running group sum (g = -1: running sum without the offset term)
  float4v db;      // offset term of the running sum, g = -1 only
#pragma unroll
  for (int rr = 0; rr < R; rr++) {
    acc[rr] = float4v{0.f, 0.f, 0.f, 0.f};
    d[rr] = float4v{0.f, 0.f, 0.f, 0.f};
  }
  db = float4v{0.f, 0.f, 0.f, 0.f};
  _Float16 zrow[R];  // g = -1: zero of this lane's row
  if constexpr (!GROUPED && ZP) {
#pragma unroll
    for (int rr = 0; rr < R; rr++)
      zrow[rr] = live ? storage_to_half(a.zeros[(size_t)(rb0 + rr) * 16 + r16]) : (_Float16)128.0f;
  }

  auto fold = [&](const uint2 s4, int rr, const float4v v) {
    const uint16_t sb[4] = {(uint16_t)s4.x, (uint16_t)(s4.x >> 16), (uint16_t)s4.y, (uint16_t)(s4.y >> 16)};
#pragma unroll
    for (int i = 0; i < 4; i++) acc[rr][i] += storage_to_float(sb[i]) * v[i];
  };

  const float4v zero4 = {0.f, 0.f, 0.f, 0.f};

  // constant operand -(1024 + centre * 2^p): removes the magic offset and centres the codes
  auto bias_operand = [&](auto jtag) {
    constexpr int J = decltype(jtag)::value;
    constexpr float cc = (float)Codec<BITS>::kCentre;
    Frag bias;
    bias.p[0] = h2_splat(-1024.0f) - pow_pair<BITS, J, 0>(cc);
    bias.p[1] = h2_splat(-1024.0f) - pow_pair<BITS, J, 1>(cc);
    bias.p[2] = h2_splat(-1024.0f) - pow_pair<BITS, J, 2>(cc);
    bias.p[3] = h2_splat(-1024.0f) - pow_pair<BITS, J, 3>(cc);
    return bias;
  };
  // operand -(zero - 128) / 2^(8-b) * 2^p for this lane's row: exact in fp16
  auto zero_operand = [&](_Float16 zv, auto jtag) {
    constexpr int J = decltype(jtag)::value;
    const _Float16 zrel = (_Float16)128.0f - zv;
    const half2v z2 = {zrel, zrel};
    Frag az;
    az.p[0] = z2 * pow_pair<BITS, J, 0>(1.0f / kMul);
    az.p[1] = z2 * pow_pair<BITS, J, 1>(1.0f / kMul);
    az.p[2] = z2 * pow_pair<BITS, J, 2>(1.0f / kMul);
    az.p[3] = z2 * pow_pair<BITS, J, 3>(1.0f / kMul);
    return az;
  };
  auto raw_operand = [&](const StageT& st, int u, int rr, auto jtag) {
    constexpr int J = decltype(jtag)::value;
    Frag aw;
    raw_octet<BITS, J>(st.w[u][rr], kc_unpack, aw.u);
    return aw;
  };
#define MATGPTQ_MFMA(A, B, C) __builtin_amdgcn_mfma_f32_16x16x32_f16((A).h, (B).h, (C), 0, 0, 0)

  // One tile (tl = its index inside the LDS copy of X').  The offset chain does not depend
  // on the row, so it is computed once and every row block's chain starts from it.
  auto tile_step = [&](const StageT& st, int u, int tl) {
    using J0 = std::integral_constant<int, 0>;
    using J1 = std::integral_constant<int, 1>;
    using J2 = std::integral_constant<int, 2>;
    using J3 = std::integral_constant<int, 3>;
    Frag b[4];
#pragma unroll
    for (int j = 0; j < 4; j++) b[j].v = *reinterpret_cast<const uint4*>(xb + tl * 128 + j * 32);
    if constexpr (GROUP == 128) {
      float4v t = MATGPTQ_MFMA(bias_operand(J0{}), b[0], zero4);
      t = MATGPTQ_MFMA(bias_operand(J1{}), b[1], t);
      t = MATGPTQ_MFMA(bias_operand(J2{}), b[2], t);
      t = MATGPTQ_MFMA(bias_operand(J3{}), b[3], t);
#pragma unroll
      for (int rr = 0; rr < R; rr++) {
        float4v v = MATGPTQ_MFMA(raw_operand(st, u, rr, J0{}), b[0], t);
        v = MATGPTQ_MFMA(raw_operand(st, u, rr, J1{}), b[1], v);
        v = MATGPTQ_MFMA(raw_operand(st, u, rr, J2{}), b[2], v);
        v = MATGPTQ_MFMA(raw_operand(st, u, rr, J3{}), b[3], v);
        if constexpr (ZP) {
          const _Float16 zv = st.z[u][rr][0];
          v = MATGPTQ_MFMA(zero_operand(zv, J0{}), b[0], v);
          v = MATGPTQ_MFMA(zero_operand(zv, J1{}), b[1], v);
          v = MATGPTQ_MFMA(zero_operand(zv, J2{}), b[2], v);
          v = MATGPTQ_MFMA(zero_operand(zv, J3{}), b[3], v);
        }
        fold(st.s[u][rr][0], rr, v);
      }
    } else if constexpr (GROUP == 32) {
      auto octet = [&](auto jtag) {
        constexpr int J = decltype(jtag)::value;
        const float4v t = MATGPTQ_MFMA(bias_operand(jtag), b[J], zero4);
#pragma unroll
        for (int rr = 0; rr < R; rr++) {
          float4v v = MATGPTQ_MFMA(raw_operand(st, u, rr, jtag), b[J], t);
          if constexpr (ZP) v = MATGPTQ_MFMA(zero_operand(st.z[u][rr][J], jtag), b[J], v);
          fold(st.s[u][rr][J], rr, v);
        }
      };
      octet(J0{});
      octet(J1{});
      octet(J2{});
      octet(J3{});
    } else {
      db = MATGPTQ_MFMA(bias_operand(J0{}), b[0], db);
      db = MATGPTQ_MFMA(bias_operand(J1{}), b[1], db);
      db = MATGPTQ_MFMA(bias_operand(J2{}), b[2], db);
      db = MATGPTQ_MFMA(bias_operand(J3{}), b[3], db);
#pragma unroll
      for (int rr = 0; rr < R; rr++) {
        d[rr] = MATGPTQ_MFMA(raw_operand(st, u, rr, J0{}), b[0], d[rr]);
        d[rr] = MATGPTQ_MFMA(raw_operand(st, u, rr, J1{}), b[1], d[rr]);
        d[rr] = MATGPTQ_MFMA(raw_operand(st, u, rr, J2{}), b[2], d[rr]);
        d[rr] = MATGPTQ_MFMA(raw_operand(st, u, rr, J3{}), b[3], d[rr]);
        if constexpr (ZP) {
          d[rr] = MATGPTQ_MFMA(zero_operand(zrow[rr], J0{}), b[0], d[rr]);
          d[rr] = MATGPTQ_MFMA(zero_operand(zrow[rr], J1{}), b[1], d[rr]);
          d[rr] = MATGPTQ_MFMA(zero_operand(zrow[rr], J2{}), b[2], d[rr]);
          d[rr] = MATGPTQ_MFMA(zero_operand(zrow[rr], J3{}), b[3], d[rr]);
        }
      }
    }
  };
#undef MATGPTQ_MFMA

  auto compute_stage = [&](const StageT& st, int c0, int c1, int stage) {
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int t = c0 + ws + W * (stage * U + u);
      if (t < c1) tile_step(st, u, t - c0);
    }
  };

  auto stages_of = [&](int c0, int c1) {
    const int span = c1 - c0 - ws;  // this wave owns tiles c0+ws, c0+ws+W, ... below c1
    const int my_tiles = (live && span > 0) ? (span + W - 1) / W : 0;
    return (my_tiles + U - 1) / U;
  };

  auto run_stages = [&](int c0, int c1, int n_stages) {
    if constexpr (STREAM) {
      // two stages per trip so that the prefetched stage needs no register copy.  Every trip
      // issues both loads whether or not those stages exist (a stage past the end reads through
      // zero-length descriptors): with a branch around a load the compiler has to assume the
      // fewer loads in flight of the two paths, and its wait before the current stage's first
      // use would then also wait for the stage just requested.
      for (int stage = 0; stage < n_stages; stage += 2) {
        load_stage(nxt, c0, c1, stage + 1);
        compute_stage(cur, c0, c1, stage);
        load_stage(cur, c0, c1, stage + 2);
        compute_stage(nxt, c0, c1, stage + 1);
      }
    } else {
      for (int stage = 0; stage < n_stages; stage++) {
        if (stage > 0) load_stage(cur, c0, c1, stage);
        compute_stage(cur, c0, c1, stage);
      }
    }
  };

  // M = 1: a wave reads only the activations of its own tiles (ws, ws + W, ...), so it stages
  // exactly those, 16 chunks per tile, and needs no barrier before it starts: trip j covers the
  // wave's tiles 4 XU j .. 4 XU (j+1) - 1, lane l the chunk l % 16 of tile 4 (XU j + i) + l / 16.
  // A tile beyond K repeats the wave's first tile (same value to the same place).
  auto x_fetch_own = [&](XTrip& t, int j) {
    const half8* src = reinterpret_cast<const half8*>(a.x);
#pragma unroll
    for (int i = 0; i < XU; i++) {
      const int ti = ws + W * (4 * (XU * j + i) + q);
      const int c = (ti < a.k_tiles ? ti : ws) * 16 + r16;
      t.dst[i] = c * 8;
      t.odd[i] = BITS == 2 && ((c >> 2) & 1) != 0;
      t.v[i] = src[c];
    }
  };

  XTrip xt;
  if constexpr (!CHUNKED) {
    // all of X' fits in LDS
    const int n_stages = stages_of(0, a.k_tiles);
    if (a.M == 1) {
      x_fetch_own(xt, 0);
      load_stage(cur, 0, a.k_tiles, 0);
      x_commit(xt);
      const int own = (a.k_tiles - ws + W - 1) / W;  // (W <= K / 128: every wave has a tile)
      for (int j = 1; j * 4 * XU < own; j++) {
        x_fetch_own(xt, j);
        x_commit(xt);
      }
    } else {
      x_fetch(xt, 0, a.k_tiles * 16, tid);
      load_stage(cur, 0, a.k_tiles, 0);
      stage_x(xt, 0, a.k_tiles);
      __syncthreads();
    }
    run_stages(0, a.k_tiles, n_stages);
  } else {
    // K is walked in chunks of kc tiles so that the LDS copy of X' stays small
    for (int c0 = 0; c0 < a.k_tiles; c0 += kc) {
      const int c1 = c0 + kc < a.k_tiles ? c0 + kc : a.k_tiles;
      const int n_stages = stages_of(c0, c1);
      x_fetch(xt, c0, (c1 - c0) * 16, tid);
      load_stage(cur, c0, c1, 0);
      if (c0 > 0) __syncthreads();  // all waves are done with the previous contents of X'
      stage_x(xt, c0, c1);
      __syncthreads();
      run_stages(c0, c1, n_stages);
    }
  }

  if constexpr (!GROUPED) {
    if (live) {
#pragma unroll
      for (int rr = 0; rr < R; rr++)
        fold(*reinterpret_cast<const uint2*>(a.scales + (size_t)(rb0 + rr) * 16 + 4 * q), rr, d[rr] + db);
    }
  }

  // combine the W partial sums of each slot: red[wave][rr][lane*4 + i]
#pragma unroll
  for (int rr = 0; rr < R; rr++)
    *reinterpret_cast<float4v*>(red + ((wave * R + rr) * 64 + lane) * 4) = acc[rr];
  __syncthreads();

  const int outs = a.M << sh.lg_rows;
  for (int o = tid; o < outs; o += blockDim.x) {
    const int n = o >> sh.lg_rows;
    const int rowl = o & ((1 << sh.lg_rows) - 1);
    const int rbl = rowl >> 4, row = rowl & 15;  // row block inside the workgroup
    const int sl = rbl / R, rr = rbl % R;
    const int grow = (rb_wg + rbl) * 16 + row;
    if (grow < a.N) {
      const float* src = red + ((sl * W) * R + rr) * 256 + (((row >> 2) * 16 + n) << 2) + (row & 3);
      float sum = 0.f;
      for (int w = 0; w < W; w++) sum += src[w * R * 256];
      a.y[(size_t)n * a.N + grow] = float_to_storage(sum * kMul);
    }
  }
}

// stream: up to 16 waves per workgroup, 128 VGPRs
template <int BITS, int GROUP, bool ZP, int R>
__global__ void __launch_bounds__(1024)
decode_stream_kernel(const GemmArgs a, const DecodeShape sh) {
  decode_body<BITS, GROUP, ZP, R, true, false>(a, sh);
}

// burst: up to 8 waves per workgroup; register budget of 4 waves per SIMD (128 VGPRs), which
// two resident workgroups per CU already reach
template <int BITS, int GROUP, bool ZP, int R>
__global__ void __launch_bounds__(512, 4)
decode_burst_kernel(const GemmArgs a, const DecodeShape sh) {
  decode_body<BITS, GROUP, ZP, R, false, false>(a, sh);
}

// chunked: X' staged kc tiles at a time (large M * K)
template <int BITS, int GROUP, bool ZP, int R>
__global__ void __launch_bounds__(512, 4)
decode_chunked_kernel(const GemmArgs a, const DecodeShape sh) {
  decode_body<BITS, GROUP, ZP, R, false, true>(a, sh);
}

template <int GROUP, bool ZP, int R>
hipError_t launch_one(const GemmArgs& a, int S, int W, int kc, bool stream_flavour, size_t smem,
                      hipStream_t stream) {
  const int per_wg = S * R;
  int lg = 4;
  while ((1 << lg) < per_wg * 16) lg++;
  const dim3 grid((a.row_blocks + per_wg - 1) / per_wg), block(64 * S * W);
  const DecodeShape sh{S, W, kc, lg};
  if (kc < a.k_tiles)
    hipLaunchKernelGGL((decode_chunked_kernel<kBits, GROUP, ZP, R>), grid, block, smem, stream, a, sh);
  else if (stream_flavour)
    hipLaunchKernelGGL((decode_stream_kernel<kBits, GROUP, ZP, R>), grid, block, smem, stream, a, sh);
  else
    hipLaunchKernelGGL((decode_burst_kernel<kBits, GROUP, ZP, R>), grid, block, smem, stream, a, sh);
  return hipGetLastError();
}

template <int GROUP, bool ZP>
hipError_t launch_r(const GemmArgs& a, int R, int S, int W, int kc, bool sf, size_t smem,
                    hipStream_t s) {
  if (R == 1) return launch_one<GROUP, ZP, 1>(a, S, W, kc, sf, smem, s);
  if (R == 2) return launch_one<GROUP, ZP, 2>(a, S, W, kc, sf, smem, s);
  return launch_one<GROUP, ZP, 4>(a, S, W, kc, sf, smem, s);
}

}  // namespace

// Entry of this translation unit: launch the decode kernel for bitwidth MATGPTQ_BITS.
// R in {1,2,4} row blocks per wave, S slots and W k-slices per workgroup
// (S*W <= 16 for the stream flavour, <= 8 for burst), kc = tiles of K staged in LDS at
// a time (kc < K/128 selects the chunked kernel, 8 waves at most), smem = dynamic LDS
// bytes (see decode_lds_bytes in abi.hip).
#define MATGPTQ_CAT2(a, b) a##b
#define MATGPTQ_CAT(a, b) MATGPTQ_CAT2(a, b)
#if MATGPTQ_BF16
#define MATGPTQ_LAUNCH_NAME MATGPTQ_CAT(MATGPTQ_CAT(launch_decode_b, MATGPTQ_BITS), _bf16)
#else
#define MATGPTQ_LAUNCH_NAME MATGPTQ_CAT(launch_decode_b, MATGPTQ_BITS)
#endif
hipError_t MATGPTQ_LAUNCH_NAME(const GemmArgs& a, int group_size, int R,
                                                      int S, int W, int kc, bool stream_flavour,
                                                      size_t smem, hipStream_t stream) {
  const bool zp = a.zeros != nullptr;
  if (group_size == 128)
    return zp ? launch_r<128, true>(a, R, S, W, kc, stream_flavour, smem, stream)
              : launch_r<128, false>(a, R, S, W, kc, stream_flavour, smem, stream);
  if (group_size == 32)
    return zp ? launch_r<32, true>(a, R, S, W, kc, stream_flavour, smem, stream)
              : launch_r<32, false>(a, R, S, W, kc, stream_flavour, smem, stream);
  return zp ? launch_r<-1, true>(a, R, S, W, kc, stream_flavour, smem, stream)
            : launch_r<-1, false>(a, R, S, W, kc, stream_flavour, smem, stream);
}

}  // namespace matgptq
