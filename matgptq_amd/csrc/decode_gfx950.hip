// Decode-regime kernel (M <= 16): HBM-bound product of packed b-bit codes with a
// few activation rows.  Compiled once per bitwidth with -DMATGPTQ_BITS=b.
// Role of the reference's gptq_matryoshka_simt / gptq_matryoshka at small batch
// (inference_lib/matgptq_cuda/csrc/matgptq_gemm.cu:337-953); the design is its own:
//
//  * one workgroup owns R row blocks (16 rows each) and all of K; its W waves take
//    the 128-column tiles of those rows round-robin, so each wave streams whole
//    tiles with one coalesced 16-byte load per lane and segment;
//  * codes are turned into exact fp16 integers (c - 2^(b-1)) in registers and fed
//    to v_mfma_f32_16x16x32_f16 as the 16x32 operand; the activations are the
//    32x16 operand (columns = batch rows, unused columns are zero), read from an
//    LDS copy of X when it fits and from global memory otherwise;
//  * per quantisation group the fp32 tile sum is multiplied by the group scale in
//    fp32; a general zero point costs one extra MFMA per octet against a constant
//    operand of ones (sum of x over the group) and no per-weight work;
//  * the W partial results are combined through LDS and stored as fp16.
#include "device_common.h"

#ifndef MATGPTQ_BITS
#error "compile with -DMATGPTQ_BITS={2,3,4,6,8}"
#endif

namespace matgptq {

namespace {

constexpr int kBits = MATGPTQ_BITS;

// Tiles a wave keeps in flight per pipeline stage, for R row blocks per wave.
constexpr int tiles_in_flight(int bits, int r) {
  const int u = (16 + r * bits - 1) / (r * bits);
  return u < 1 ? 1 : (u > 8 ? 8 : u);
}

template <int BITS, int R, int U, bool ZP, bool GROUPED>
struct Stage {
  uint32_t w[U][R][BITS];
  uint2 s[GROUPED ? U : 1][R][GROUPED ? 4 : 1];  // up to 4 groups per tile (g = 32)
  uint2 z[(GROUPED && ZP) ? U : 1][R][(GROUPED && ZP) ? 4 : 1];
};

template <int BITS, int GROUP, bool ZP, int R, bool XLDS>
__global__ void __launch_bounds__(512)
decode_kernel(const GemmArgs a) {
  constexpr int U = tiles_in_flight(BITS, R);
  constexpr bool GROUPED = GROUP != -1;
  constexpr int GPT = GROUP == 32 ? 4 : 1;  // groups per tile
  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int W = blockDim.x >> 6;
  const int r16 = lane & 15;  // row of the weight operand / batch column of the x operand
  const int q = lane >> 4;
  const int rb0 = blockIdx.x * R;

  float* red = reinterpret_cast<float*>(smem);                       // [W][R][256]
  _Float16* xs = reinterpret_cast<_Float16*>(smem + W * R * 1024);   // [M][K + 8]
  const int pitch = a.K + 8;

  const int my_tiles = (a.k_tiles - wave + W - 1) / W;  // tiles wave, wave+W, ...
  const int n_stages = (my_tiles + U - 1) / U;

  const size_t tile_stride = (size_t)tile_words(BITS);
  const uint32_t* wbase = a.packed + (size_t)rb0 * a.k_tiles * tile_stride;
  const size_t rb_stride = (size_t)a.k_tiles * tile_stride;

  auto load_stage = [&](Stage<BITS, R, U, ZP, GROUPED>& st, int stage) {
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int t = wave + W * (stage * U + u);
      if (t < a.k_tiles) {
#pragma unroll
        for (int rr = 0; rr < R; rr++) {
          load_tile_words<BITS>(wbase + rr * rb_stride + (size_t)t * tile_stride, lane, st.w[u][rr]);
          if constexpr (GROUPED) {
#pragma unroll
            for (int gg = 0; gg < GPT; gg++) {
              const size_t so = ((size_t)(rb0 + rr) * a.G + (size_t)t * GPT + gg) * 16 + 4 * q;
              st.s[u][rr][gg] = *reinterpret_cast<const uint2*>(a.scales + so);
              if constexpr (ZP) st.z[u][rr][gg] = *reinterpret_cast<const uint2*>(a.zeros + so);
            }
          }
        }
      }
    }
  };

  Stage<BITS, R, U, ZP, GROUPED> cur, nxt;
  if (n_stages > 0) load_stage(cur, 0);

  if constexpr (XLDS) {
    const int chunks_per_row = a.K >> 3;
    const int total = a.M * chunks_per_row;
    for (int i = tid; i < total; i += blockDim.x) {
      const int m = i / chunks_per_row, c = i - m * chunks_per_row;
      const uint4 v = reinterpret_cast<const uint4*>(a.x + (size_t)m * a.K)[c];
      *reinterpret_cast<uint4*>(xs + m * pitch + c * 8) = v;
    }
    __syncthreads();
  }

  float4v acc[R];   // sum over groups of scale * group sum (grouped), unused otherwise
  float4v d[R];     // running MFMA sum of (c - centre) * x
  float4v d2;       // running MFMA sum of x (zero-point term)
#pragma unroll
  for (int rr = 0; rr < R; rr++) {
    acc[rr] = float4v{0.f, 0.f, 0.f, 0.f};
    d[rr] = float4v{0.f, 0.f, 0.f, 0.f};
  }
  d2 = float4v{0.f, 0.f, 0.f, 0.f};

  Frag ones;
  ones.u[0] = ones.u[1] = ones.u[2] = ones.u[3] = 0x3C003C00u;

  constexpr float kMul = (float)(1 << (8 - BITS));
  constexpr float kInvMul = 1.0f / kMul;

  // acc += scale * (d - (zero - 128) / 2^(8-b) * d2); the common factor 2^(8-b) is applied at the end
  auto fold_group = [&](const Stage<BITS, R, U, ZP, GROUPED>& st, int u, int gg) {
#pragma unroll
    for (int rr = 0; rr < R; rr++) {
      H4 s;
      s.v = st.s[u][rr][gg];
      H4 z;
      if constexpr (ZP) z.v = st.z[u][rr][gg];
#pragma unroll
      for (int i = 0; i < 4; i++) {
        float t = d[rr][i];
        if constexpr (ZP) t -= ((float)z.h[i] - 128.0f) * kInvMul * d2[i];
        acc[rr][i] += (float)s.h[i] * t;
        d[rr][i] = 0.f;
      }
    }
    if constexpr (ZP) d2 = float4v{0.f, 0.f, 0.f, 0.f};
  };

  auto octet_step = [&](const Stage<BITS, R, U, ZP, GROUPED>& st, int u, int t, auto jtag) {
    constexpr int J = decltype(jtag)::value;
    Frag b;
    b.v = make_uint4(0u, 0u, 0u, 0u);
    if (r16 < a.M) {
      const int kk = t * 128 + J * 32 + q * 8;
      if constexpr (XLDS)
        b.v = *reinterpret_cast<const uint4*>(xs + r16 * pitch + kk);
      else
        b.v = *reinterpret_cast<const uint4*>(a.x + (size_t)r16 * a.K + kk);
    }
#pragma unroll
    for (int rr = 0; rr < R; rr++) {
      Frag aw;
      centred_octet<BITS, J>(st.w[u][rr], aw);
      d[rr] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aw.h, b.h, d[rr], 0, 0, 0);
    }
    if constexpr (ZP) d2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones.h, b.h, d2, 0, 0, 0);
    if constexpr (GROUP == 32) fold_group(st, u, J);
  };

  for (int stage = 0; stage < n_stages; stage++) {
    if (stage + 1 < n_stages) load_stage(nxt, stage + 1);
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int t = wave + W * (stage * U + u);
      if (t < a.k_tiles) {
        octet_step(cur, u, t, std::integral_constant<int, 0>{});
        octet_step(cur, u, t, std::integral_constant<int, 1>{});
        octet_step(cur, u, t, std::integral_constant<int, 2>{});
        octet_step(cur, u, t, std::integral_constant<int, 3>{});
        if constexpr (GROUP == 128) fold_group(cur, u, 0);
      }
    }
    if (stage + 1 < n_stages) cur = nxt;
  }

  if constexpr (!GROUPED) {
    // one scale (and zero) per row: fold once
#pragma unroll
    for (int rr = 0; rr < R; rr++) {
      const size_t so = (size_t)(rb0 + rr) * 16 + 4 * q;
      H4 s, z;
      s.v = *reinterpret_cast<const uint2*>(a.scales + so);
      if constexpr (ZP) z.v = *reinterpret_cast<const uint2*>(a.zeros + so);
#pragma unroll
      for (int i = 0; i < 4; i++) {
        float t = d[rr][i];
        if constexpr (ZP) t -= ((float)z.h[i] - 128.0f) * kInvMul * d2[i];
        acc[rr][i] = (float)s.h[i] * t;
      }
    }
  }

  // combine the W partial sums: red[wave][rr][lane*4 + i]
#pragma unroll
  for (int rr = 0; rr < R; rr++)
    *reinterpret_cast<float4v*>(red + ((wave * R + rr) * 64 + lane) * 4) = acc[rr];
  __syncthreads();

  const int outs = R * 16 * a.M;
  for (int o = tid; o < outs; o += blockDim.x) {
    const int n = o / (R * 16);
    const int rowl = o - n * (R * 16);
    const int rr = rowl >> 4, row = rowl & 15;
    const int idx = (((row >> 2) * 16 + n) << 2) + (row & 3);
    float sum = 0.f;
    for (int w = 0; w < W; w++) sum += red[(w * R + rr) * 256 + idx];
    const _Float16 h = (_Float16)(sum * kMul);
    reinterpret_cast<_Float16*>(a.y)[(size_t)n * a.N + (size_t)(rb0 + rr) * 16 + row] = h;
  }
}

template <int GROUP, bool ZP, int R, bool XLDS>
hipError_t launch_one(const GemmArgs& a, int W, size_t smem, hipStream_t stream) {
  const dim3 grid(a.row_blocks / R), block(64 * W);
  hipLaunchKernelGGL((decode_kernel<kBits, GROUP, ZP, R, XLDS>), grid, block, smem, stream, a);
  return hipGetLastError();
}

template <int GROUP, bool ZP>
hipError_t launch_rx(const GemmArgs& a, int R, int W, bool xlds, size_t smem, hipStream_t s) {
  if (xlds) {
    if (R == 1) return launch_one<GROUP, ZP, 1, true>(a, W, smem, s);
    if (R == 2) return launch_one<GROUP, ZP, 2, true>(a, W, smem, s);
    return launch_one<GROUP, ZP, 4, true>(a, W, smem, s);
  }
  if (R == 1) return launch_one<GROUP, ZP, 1, false>(a, W, smem, s);
  if (R == 2) return launch_one<GROUP, ZP, 2, false>(a, W, smem, s);
  return launch_one<GROUP, ZP, 4, false>(a, W, smem, s);
}

}  // namespace

// Entry of this translation unit: launch the decode kernel for bitwidth MATGPTQ_BITS.
// R in {1,2,4} row blocks per workgroup, W in {1..8} waves, xlds: stage X in LDS.
#define MATGPTQ_CAT2(a, b) a##b
#define MATGPTQ_CAT(a, b) MATGPTQ_CAT2(a, b)
hipError_t MATGPTQ_CAT(launch_decode_b, MATGPTQ_BITS)(const GemmArgs& a, int group_size,
                                                      int R, int W, bool xlds,
                                                      hipStream_t stream) {
  const bool zp = a.zeros != nullptr;
  const size_t smem = (size_t)W * R * 1024 + (xlds ? (size_t)a.M * (a.K + 8) * 2 : 0);
  if (group_size == 128)
    return zp ? launch_rx<128, true>(a, R, W, xlds, smem, stream)
              : launch_rx<128, false>(a, R, W, xlds, smem, stream);
  if (group_size == 32)
    return zp ? launch_rx<32, true>(a, R, W, xlds, smem, stream)
              : launch_rx<32, false>(a, R, W, xlds, smem, stream);
  return zp ? launch_rx<-1, true>(a, R, W, xlds, smem, stream)
            : launch_rx<-1, false>(a, R, W, xlds, smem, stream);
}

}  // namespace matgptq
