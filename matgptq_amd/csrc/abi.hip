// C ABI entry points: argument checks, kernel selection, launches.
// Counterpart of the reference's host launcher and dispatch macros
// (inference_lib/matgptq_cuda/csrc/matgptq_gemm.cu:955-1065); it returns error
// codes where the reference prints and exits (include/common.cuh:44-51).
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>
#include <mutex>

#include "../../include/matgptq_abi.h"
#include "device_common.h"
#include "prefill_plan.h"

// Scratch of matgptq_gemm_master_static: device memory that lives in the library's code object, so
// that entry point needs no allocation at all.  One copy per GPU, at its own address.
constexpr size_t kStaticScratchBytes = (size_t)MATGPTQ_STATIC_WORKSPACE_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace matgptq {

int check_problem(int bits, int group_size, int64_t N, int64_t K);  // pack_host.cpp

#define MATGPTQ_DECL(B)                                                                        \
  hipError_t launch_decode_b##B(const GemmArgs&, int group_size, int R, int S, int W, int kc,  \
                                bool stream_flavour, size_t smem, hipStream_t);                \
  hipError_t launch_prefill_b##B(const GemmArgs&, int group_size, int cfg, hipStream_t);          \
  hipError_t launch_skinny_b##B(const GemmArgs&, int group_size, int r, int mb, bool master, hipStream_t);   \
  hipError_t launch_gemv_b##B(const GemmArgs&, int group_size, int shape, int W, size_t lds_pad, bool master, hipStream_t);  \
  hipError_t launch_gemv_b##B##_bf16(const GemmArgs&, int group_size, int shape, int W, size_t lds_pad, bool master, hipStream_t); \
  hipError_t launch_gemv_prologue_b##B(const GemmArgs&, int kind, int shape, int W, const void* b, const void* w, void* out, \
                                       float eps, hipStream_t);                                                            \
  hipError_t launch_skinny_b##B##_bf16(const GemmArgs&, int group_size, int r, int mb, bool master, hipStream_t); \
  hipError_t launch_decode_b##B##_bf16(const GemmArgs&, int group_size, int R, int S, int W,   \
                                       int kc, bool stream_flavour, size_t smem, hipStream_t); \
  hipError_t launch_prefill_b##B##_bf16(const GemmArgs&, int group_size, int cfg, hipStream_t);
MATGPTQ_DECL(2)
MATGPTQ_DECL(3)
MATGPTQ_DECL(4)
MATGPTQ_DECL(6)
MATGPTQ_DECL(8)
#undef MATGPTQ_DECL

hipError_t launch_pack(const uint8_t*, int64_t, int64_t, int, int, uint32_t*, hipStream_t);
hipError_t launch_unpack(const uint32_t*, int64_t, int64_t, int, uint8_t*, hipStream_t);
hipError_t launch_slice(const uint8_t*, int64_t, int, uint8_t*, hipStream_t);
hipError_t launch_pack_master(const uint8_t*, int64_t, int64_t, uint32_t*, hipStream_t);
hipError_t launch_master_slice(const uint32_t*, int64_t, int64_t, int, bool, void*, hipStream_t);
hipError_t launch_reorder(const uint16_t*, int64_t, int64_t, uint16_t*, hipStream_t);
hipError_t launch_tail_gemm(int bits, bool bf16, const GemmArgs&, int group_size, hipStream_t);
hipError_t launch_read_probe(const void*, size_t, hipStream_t);
hipError_t launch_dequant(int, int, int64_t, int64_t, const uint32_t*, const uint16_t*,
                          const uint16_t*, uint16_t*, hipStream_t);

namespace {

constexpr int kDecodeMaxM = 16;
constexpr int kGemvMaxM = 4;
constexpr int kGemvEightMaxM = 8;  // its instantiation for five to eight batch rows (group sizes 128 and -1)
// (tiles per wave and round, row blocks per workgroup) of the gemv kernel's instantiations
// (group sizes 32 and -1 and the master-resident planes: entries 1 and 2 only)
constexpr int kNumGemvShapes = 7;
constexpr int kGemvShapes[kNumGemvShapes][2] = {{8, 1}, {4, 1}, {4, 2}, {2, 2}, {2, 4}, {2, 1}, {4, 4}};
constexpr size_t kLdsBudget = 64 * 1024;  // dynamic LDS a decode workgroup may ask for

struct Plan {
  bool gemv;     // batch 1..4 at group 128: gemv kernel, `shape` = its (T, R) entry, W waves
  int shape;
  size_t pad;    // gemv: dynamic LDS to ask for at least (bounds the workgroups per CU)
  bool decode;
  bool skinny;   // mid-batch kernel (K split inside the workgroup), R row blocks per workgroup
  int mb;        // mid-batch: blocks of 16 batch rows per workgroup
  int R, S, W;   // decode: row blocks per wave, slots and k-slices per workgroup
  int kc;        // decode: tiles of K staged in LDS at a time
  bool stream;   // decode: double-buffered flavour
  size_t smem;   // decode: dynamic LDS bytes
  int cfg;       // prefill: tile configuration
};

// (slots, k-slices) per workgroup selectable through the variant override
constexpr int kNumShapes = 14;
constexpr int kShapes[kNumShapes][2] = {{1, 8}, {1, 4}, {2, 4}, {2, 2}, {4, 2}, {4, 1}, {8, 1},
                                        {1, 2}, {2, 1}, {1, 16}, {2, 8}, {4, 4}, {8, 2}, {1, 1}};

// LDS of a decode workgroup: partial sums (1 KiB per wave and row block) and kc tiles
// of activations.
size_t decode_lds_bytes(int R, int S, int W, int kc, int64_t M) {
  return (size_t)S * W * R * 1024 + (size_t)M * ((size_t)kc * 128 + 8) * 2;
}

// Automatic choice; the flags word can override it for benchmarks:
//   bits 8..15 : 0 = automatic, 1 + rsel + 3*shape = decode (rsel: R = 1,2,4; shape: kShapes),
//                64 + cfg = prefill tile configuration 0..15, 89 and 90 = configurations 16 and 17,
//                80 + rsel + 3*msel = mid-batch kernel (rsel: R = 1,2,4; msel: 16, 32, 64 batch rows),
//                91 = mid-batch kernel with R = 8 and 32 batch rows
//   bits 16..17: decode flavour, 0 = automatic, 1 = burst, 2 = stream
int make_plan(int bits, int group_size, int64_t N, int64_t K, int64_t M, bool zp, uint32_t flags,
              Plan* p) {
  const int row_blocks = (int)(N / 16), k_tiles = (int)(K / 128);
  const int variant = (int)((flags & MATGPTQ_FLAG_VARIANT_MASK) >> MATGPTQ_FLAG_VARIANT_SHIFT);
  const int flavour = (int)((flags >> 16) & 3u);
  p->decode = M <= kDecodeMaxM;
  p->gemv = false;
  p->shape = 0;
  p->pad = 0;
  p->skinny = false;
  p->mb = 2;
  p->cfg = 0;
  // default decode shape (measured on MI355X, M = 1, Llama-3-8B layers): eight waves per
  // workgroup, all of them splitting K; four row blocks per wave once there are enough
  // row blocks to keep every CU busy that way
  int W = 8, S = 1;
  while (W > 1 && W > k_tiles) { W >>= 1; S <<= 1; }
  // (group 32 carries four scales and zeros per tile and row block: two row blocks at most)
  int R = row_blocks >= 1024 ? (group_size == 32 ? 2 : 4) : 1;
  // from four batch rows on, the copy of X' each workgroup stages starts to count: more row
  // blocks per workgroup (two slots of two, or two per wave) amortise it better
  if (M >= 4 && k_tiles >= 8) {
    if (row_blocks >= 1024) { R = 2; S = 2; W = 4; }
    else if (row_blocks >= 320) { R = 2; }
  }
  // (four row blocks per mid-batch workgroup only up to 6 bits and one scale per tile: registers)
  const int r_max = group_size == 32 || bits > 6 ? 2 : 4;
  // (eight: pre-sliced codes up to 4 bits with one scale per tile or row, 32 batch rows per workgroup)
  const bool eight_rows = group_size != 32 && bits <= 4;
  // row blocks per mid-batch workgroup: as many as still leave about 160 workgroups (the
  // activations are re-read once per workgroup column)
  auto mid_rows = [&](int64_t m_tiles) {
    for (int r = r_max; r > 1; r >>= 1)
      if ((int64_t)((row_blocks + r - 1) / r) * m_tiles >= 160) return r;
    return 1;
  };
  if (!p->decode) {
    // M > 16.  The 128 x 256 tile (two waves per SIMD, activations copied straight into LDS)
    // once its workgroups fill more than half of the 512 resident slots (measured on MI355X,
    // Llama-3-8B and 70B layers).
    const int64_t wgs_big = ((N + 255) / 256) * ((M + 127) / 128);
    // the 32 x 128 staged tile: 0.95 us per K tile and round of 512 workgroups, a last partial round
    // counting as 0.35 of one at least (bf16 storage 1.2 times that, group size 32 - four scales and
    // zeros per tile - 1.4 times)
    const int64_t wgs_32 = ((N + 127) / 128) * ((M + 31) / 32);
    const double rest_32 = (double)(wgs_32 % 512) / 512.0;
    const double t_32 = 0.95 * ((flags & MATGPTQ_FLAG_BF16) ? 1.2 : 1.0) * (group_size == 32 ? 1.4 : 1.0) * (double)k_tiles *
                        (wgs_32 <= 512 ? 1.0 : (double)(wgs_32 / 512) + (rest_32 == 0.0 ? 0.0 : rest_32 < 0.35 ? 0.35 : rest_32));
    // A layer with very many rows fills the 128 x 256 tiles' slots at any batch size, but up to 64 batch
    // rows those tiles are mostly padding: a round of them costs 11.5 us + 3.2 per K tile (128256 x 4096 at
    // M = 32: 117 us, against 65 on the small tile).
    const bool small_batch_many_rows =
        M <= 64 && t_32 < (11.5 + 3.2 * (double)k_tiles) * (wgs_big > 512 ? (double)wgs_big / 512.0 : 1.0);
    if (wgs_big > 256 && small_batch_many_rows) {
      p->cfg = 4;
    } else if (wgs_big > 256) {
      p->cfg = 0;
      // Whole rounds of 512 resident workgroups plus at most half a round: the rows of that
      // fraction go to 128 x 128 tiles, which run last, one per CU, in about a third of a
      // round's time (Llama-3-70B qkv at M = 2048, 640 tiles: 355 -> 305 us).
      const int m_tiles = (int)((M + 127) / 128);
      const int nb = prefill_tail_big_tiles(row_blocks, m_tiles);
      const int64_t rest = (int64_t)((row_blocks - nb * 16 + 15) / 16) * m_tiles;
      // (one whole round only: behind three rounds the plain tile's fourth, half empty, costs less than
      // the narrow tiles do - 57344 x 8192 at M = 1024: 752 against 771 us)
      if (nb > 0 && rest > 0 && rest <= 256 && (int64_t)nb * m_tiles <= 512) p->cfg = 8;
      // When those narrow tiles number no more than the CUs, workgroups of eight waves do better: the
      // wide tiles two to a workgroup, each narrow tile with K split over two groups of four waves, so
      // that the last part of the launch runs two waves per SIMD as well (10240 x 8192 at M = 2048:
      // 285 -> 276 us with zero points, 278 -> 271 without).
      if (p->cfg == 8 && 2 * rest <= 256) p->cfg = 12;
      // Where the rows behind the whole rounds make up (nearly) one round of 128 x 192 tiles - and so would
      // be three quarters of a round of the wide tile, or more than a round of 128 x 128 tiles - they run
      // as those (57344 x 8192 at M = 512: 387 against 398 us).
      if (p->cfg == 0 && nb > 0 && m_tiles <= 512) {
        const int slots = 512 / m_tiles;
        const int rest_rb = row_blocks - nb * 16;
        const int n192 = (rest_rb + 11) / 12;
        if (rest_rb > 8 * slots && n192 <= slots && 10 * n192 >= 9 * slots) p->cfg = 15;
      }
      // Behind ONE whole round, the cheapest of the three tails, in units of a round of the wide tile:
      // a tile takes its share of the width, times 1.3 (128 rows) or 1.07 (192 rows) for the narrower
      // tile's lower rate; workgroups that number no more than the CUs sit alone there and finish in 0.7
      // of that, and 128-row tiles that few run K split in 0.35 (28672 x 4096, behind 105 us for the
      // whole round: M = 768, 162 / 324 / 216 workgroups, 180 / 176 / 162 us; M = 896, 273 / 546 / 364,
      // 212 / 215 / 193 us; M = 640, 50 / 100 / 70, 170 / 140 (K split) / 157 us).
      if (nb > 0 && (int64_t)nb * m_tiles <= 512 && row_blocks > nb * 16 && p->cfg != 12) {
        const int rest_rb = row_blocks - nb * 16;
        auto occupancy = [](int64_t n) { return n <= 256 ? 0.7 : (double)((n + 511) / 512); };
        const int64_t n256 = (int64_t)((rest_rb + 15) / 16) * m_tiles, n128 = (int64_t)((rest_rb + 7) / 8) * m_tiles;
        const int64_t n192 = (int64_t)((rest_rb + 11) / 12) * m_tiles;
        const double t256 = occupancy(n256), t128 = occupancy(n128) * 0.5 * 1.3, t192 = occupancy(n192) * 0.75 * 1.07;
        p->cfg = t192 < t256 && t192 < t128 ? 15 : t128 < t256 ? 8 : 0;
      }
      // 6-bit codes for four row blocks do not fit beside the accumulators of the 128 x 256 tile even
      // with a single set refilled octet by octet (as 8-bit codes are): it spills and runs at half the
      // rate of the 128 x 128 ring tile (8192 x 8192, M = 2048, 6 bits: 596 against 281 us).
      // Between the two, a 128 x 192 tile (three row blocks per wave) fits the registers and runs
      // about 9 % faster per weight than the 128 x 128 tile where its tiles fill the rounds of 512
      // resident workgroups as well (57344 x 8192, 6 bits: 1748 against 1906 us; on 8192 rows, 43
      // tiles of 192, it only ties).  Rounds times tile width decide.
      // bf16 storage dequantises through fp32 for the bf16 matrix instruction (four vector
      // instructions per pair of weights instead of three).  At 2 and 4 bits, and at 8 bits with one
      // scale per row, the 128 x 256 tile holds that in registers and the rules of fp16 storage apply
      // (M = 2048, 4 bits: 8192 x 8192 228 against 256 us on 128 x 128 tiles, 8192 x 28672 761 against 870,
      // 57344 x 8192 1542 against 1611 on 128 x 192).  At 3 and 6 bits, with group size 32, and at 8 bits
      // with a scale and zero per tile it spills (8 bits, 8192 x 8192: 511 us): those take the
      // 128 x 128 tile or, except at 6 bits, the 128 x 192 tile where its rounds pay.  8-bit codes fit
      // the 128 x 256 tile again once eight waves halve K between them, up to two rounds of one such
      // workgroup per CU (8192 x 8192, M = 2048: 243 against 270 us; 8192 x 28672: 889 against 1018).
      // Group size 32 with zero points keeps four scales and four zeros per tile and row block in
      // two register sets: the 128 x 256 tile spills (8192 x 8192, M = 2048: 489 us at 4 bits, 3023 us
      // at 8 bits, against 290 and 307 us on the 128 x 128 tile); the 128 x 192 tile fits up to 4 bits
      // and at 8 (57344 x 8192, 4 bits: 1728 against 1902 us).
      const bool bf16 = (flags & MATGPTQ_FLAG_BF16) != 0;
      const bool g32zp = group_size == 32 && zp;
      const int64_t wgs_192 = ((N + 191) / 192) * m_tiles, wgs_128 = ((N + 127) / 128) * m_tiles;
      const bool fits_192 = !(bf16 && (bits == 6 || group_size == 32)) && !(bits == 6 && g32zp);
      const bool bf16_narrow =
          bf16 && (group_size == 32 || !(bits == 2 || bits == 4 || (bits == 8 && group_size == -1)));
      if (bits == 6 || bf16_narrow || g32zp) {
        // (whole rounds of 512 resident workgroups up to two; beyond, the rounds blur into each other)
        auto rounds = [](int64_t w) { return w <= 1024 ? (double)((w + 511) / 512) : (double)w / 512.0 + 0.5; };
        const double t_192 = rounds(wgs_192) * 1.5 / 1.09;
        const double t_128 = rounds(wgs_128);
        p->cfg = t_192 < t_128 && fits_192 ? 9 : 3;
        if (p->cfg == 3 && bf16 && bits == 8 && group_size != 32 && wgs_big <= 512) p->cfg = 11;
        // 6-bit codes on fp16 storage with one scale per tile or row: one register set refilled octet by
        // octet fits the 128 x 256 tile once the compiler is left to order the step itself (243 registers;
        // with the ordering hints of the other widths it spilled).  Its four instructions per pair of
        // weights keep it at 41-43 % of peak, just ahead of the narrower tiles where its tiles fill whole
        // rounds (M = 2048: 8192 x 8192 263 against 265 us, 8192 x 28672 890 against 923).
        if (bits == 6 && !bf16 && group_size != 32) {
          const double t_256 = rounds(wgs_big) * 2.0 * 0.97;
          if (t_256 < t_128 && (p->cfg == 3 || t_256 < t_192)) p->cfg = 0;
        }
      } else if (wgs_192 <= 512 && fits_192) {
        // Fewer than 512 of the 128 x 256 tiles leave half of the CUs with one workgroup where the
        // kernel is built for two; 128 x 192 tiles that still fit one round of 512 spread the same
        // rows over more of the slots (M = 2048, 4 bits: 6144 x 4096 92 against 98 us, 5120 x 4096 83
        // against 91, 4608 x 3584 68 against 80; the same at 2, 3 and 8 bits).  Past 512 of them a
        // second round starts and the 128 x 256 tile is ahead again (6144 x 4096, M = 2560: 139
        // against 108 us).
        p->cfg = 9;
        // ... and where those leave slots empty while 128 x 128 tiles would need a second round, both
        // widths in one launch take every slot once (10240 x 8192 at M = 1024: 432 tiles of 192 rows on
        // 512 slots; 256 of them and 256 of 128 rows instead)
        // (the wide tiles of the mix must not number more than the CUs, or some CUs get two of them and
        // finish no earlier than with 128 x 192 tiles alone: 28672 x 4096 at M = 384, 324 wide tiles: 93
        // against 89 us)
        int narrow = 0;
        const int wide = prefill_mix_wide_tiles(row_blocks, m_tiles, &narrow);
        if (wide > 0 && wide * m_tiles <= 256) p->cfg = 14;
      } else if (wgs_big <= 512 && fits_192 && p->cfg == 0) {
        // One round of the 128 x 256 tile that leaves slots empty, while 128 x 192 tiles would need a
        // second round: both widths in one launch, a wide and a narrow tile on every CU (28672 x 4096 at
        // M = 512: 448 wide tiles on 512 slots 122 us, 256 wide and 256 narrow 104).
        int narrow = 0;
        const int wide = prefill_mix_widest_tiles(row_blocks, m_tiles, &narrow);
        if (wide > 0 && wide * m_tiles <= 256) p->cfg = 17;
      }
    } else {
      // Below that, the cheapest of four by a cost model fitted to measurements on MI355X
      // (4 bits, Llama-3-8B and 70B layers, M = 17 .. 1024), in microseconds:
      //   128 x 128 tile  1.55 per K tile, up to 2.0 as a second workgroup joins a CU,
      //                   proportionally more beyond the 512 resident slots;
      //   32 x 128 tile   as above;
      //   mid-batch kernel with 32 or 64 batch rows per workgroup: 2 + rounds x (3.5 + K tiles x
      //                   0.85 (0.12 + 0.016 R MB)), one workgroup per CU and round.
      const double kt = (double)k_tiles;
      const int64_t wgs_128 = ((N + 127) / 128) * ((M + 127) / 128);
      const double second = wgs_128 <= 256 ? 0.0 : wgs_128 >= 512 ? 1.0 : (double)(wgs_128 - 256) / 256.0;
      const double t_128 = kt * (1.55 + 0.45 * second) * (wgs_128 > 512 ? (double)wgs_128 / 512.0 : 1.0);
      p->cfg = t_128 < t_32 ? 3 : 4;
      // Where the 128 x 128 ring tiles would sit one per CU (it is built for two, whose waves cover
      // each other's waits), the staged 64 x 256 tile - twice the row blocks per dequantised
      // activation block, as many workgroups - is faster while its own workgroups fit one round
      // (M = 512: 8192 x 8192 92 against 103 us, 8192 x 28672 297 against 370; 28672 x 4096 at M = 128: 48
      // against 55).  fp16 storage, group sizes 128 and -1 (its registers hold no more).
      const int64_t wgs_64 = ((N + 255) / 256) * ((M + 63) / 64);
      if (p->cfg == 3 && wgs_128 <= 256 && wgs_64 <= 256 && wgs_64 >= 128 && group_size != 32 &&
          !(flags & MATGPTQ_FLAG_BF16))
        p->cfg = 2;
      double best = t_128 < t_32 ? t_128 : t_32;
      // Ring tiles that sit one per CU run K in two halves inside a workgroup of eight waves (two
      // per SIMD, as two workgroups would bring): 128 x 128 while those tiles number at most the
      // CUs, 3 us + 0.74 .. 0.98 per K tile, more as more of the CUs are taken (M = 512: 8192 x 8192 66
      // against 87 us on the staged 64 x 256 tile, 8192 x 28672 249 against 298; 4096 x 4096 at M = 1024 40 against 48); 128 x 256 where
      // only these number at most the CUs, 5 us + 1.4 .. 1.65 per K tile (8192 x 8192 at M = 1024 111
      // against 125 us on 128 x 128 tiles two per CU, 8192 x 28672 366 against 440), for the formats
      // whose registers fit that tile (bf16 storage: all but 3 and 6 bits and group size 32 -
      // 8192 x 8192 at M = 1024 116 against 128 us at 4 bits, 127 against 148 at 8).
      const bool bf16 = (flags & MATGPTQ_FLAG_BF16) != 0;
      if (wgs_128 <= 256) {
        const double wide_codes = bits == 8 ? 1.1 : 1.0;  // (8-bit codes: 24 against 22 us per 32 K tiles)
        const double t = 3.0 + kt * wide_codes * (0.66 + 0.32 * (double)wgs_128 / 256.0);
        if (t < best) { best = t; p->cfg = 10; }
        // ... and 64 x 128 tiles the same way where twice as many workgroups still number at most the
        // CUs, 4.5 us + 0.5 .. 0.64 per K tile (4096 x 4096 at M = 512: 25 against 30 us, 4096 x 14336:
        // 74 against 88; 6144 x 4096 at M = 256: 25 against 31)
        const int64_t wgs_64s = ((N + 127) / 128) * ((M + 63) / 64);
        const double t6 = 4.5 + kt * (bits == 8 ? 1.2 : 1.0) * (bf16 ? 1.05 : 1.0) * (0.45 + 0.19 * (double)wgs_64s / 256.0);
        if (wgs_64s <= 256 && t6 < best) { best = t6; p->cfg = 16; }
      } else if (wgs_big <= 256 && bits != 6 && !(bf16 && (bits == 3 || group_size == 32)) && !(group_size == 32 && zp)) {
        const double t = 5.0 + kt * (wgs_big > 192 ? 1.65 : 1.4);
        if (t < best) { best = t; p->cfg = 11; }
        // the same with 128 x 192 tiles where those fill more of the CUs in their one round
        // (10240 x 8192 at M = 512: 216 workgroups, 91 us against 94 on 160 of the wider tile)
        const int64_t wgs_192s = ((N + 191) / 192) * ((M + 127) / 128);
        const double t3 = 4.0 + kt * (wgs_192s > 192 ? 1.36 : 1.22);
        if (wgs_192s <= 256 && t3 < best) { best = t3; p->cfg = 13; }
      }
      for (int mb = 2; mb <= (M > 32 ? 4 : 2); mb <<= 1) {
        const int64_t m_tiles = (M + 16 * mb - 1) / (16 * mb);
        int r = mid_rows(m_tiles);
        // Eight row blocks with 32 batch rows (one workgroup per CU) where that still leaves 200
        // workgroups: the activations are copied half as often (M = 32: 28672 x 4096 21.4 against 21.9 us
        // at 4 bits, 19.3 against 21.9 at 2; 57344 x 8192 61 against 66, 57 against 65)
        if (mb == 2 && eight_rows && (int64_t)((row_blocks + 7) / 8) * m_tiles >= 200) r = 8;
        const int64_t wgs = (int64_t)((row_blocks + r - 1) / r) * m_tiles;
        // One workgroup per CU and round.  (With 32 batch rows and at most two row blocks a second
        // one fits, but two together take 1.6 times as long as one: 0.8 of the cost per tile each.)
        // 8-bit codes cost 1.1 times as much per tile, bf16 storage (weights formed in fp32) 1.05
        // times.
        const int64_t slots = 256;
        // (eight row blocks: 1.3 times the cost their count suggests - 0.41 .. 0.5 us per K tile measured)
        const double per_tile = 0.85 * (0.12 + 0.016 * r * mb) * (mb == 2 && r <= 2 ? 0.8 : 1.0) * (r == 8 ? 1.3 : 1.0) *
                                (bits == 8 ? 1.1 : 1.0) * (bf16 ? 1.05 : 1.0);
        const int64_t rounds = (wgs + slots - 1) / slots;
        // (More than a thousand batch rows in more than one round: every XCD then streams most of
        // the activations through its 4 MB of L2 once per round, and the small staged tile is ahead -
        // 1024 x 4096 at M = 2048: 51 against 34 us, 1024 x 14336: 135 against 105, 512 x 8192 at M = 4096:
        // 86 against 65.)
        if (M > 1024 && rounds > 1) continue;
        const double t = 2.0 + (double)rounds * (3.5 + kt * per_tile);
        if (t < best) {
          best = t;
          p->skinny = true;
          p->mb = mb;
          R = r;
        }
      }
    }
  } else if (flavour == 0 && M > kGemvMaxM &&
             !(bits == 8 && group_size != 32 && !(flags & MATGPTQ_FLAG_BF16) && row_blocks >= 1024)) {
    // Five to sixteen batch rows (one to four go to the gemv kernel below, and five to eight on
    // layers with few row blocks): every decode
    // workgroup stages the whole batch of activations (scaled copies, written by the vector
    // ALU), which grows with M and K, while the mid-batch kernel copies them into LDS
    // asynchronously.  Measured on MI355X (Llama-3-8B layers, 2, 4 and 8 bits, M = 5 .. 16, weights
    // cold): the mid-batch kernel wins everywhere (M = 7, 4 bits: 4096 x 4096 5.4 against 7.3 us,
    // 6144 x 4096 6.1 against 8.5, 28672 x 4096 15.8 against 20.4; group size 32 at 6 and 8 bits,
    // M = 8: 23.3 and 23.7 against 33.8 and 29.0; bf16 storage at 8 bits 21.7 against 25.2) except at
    // 8 bits on fp16 storage with one scale per tile or row, on layers with many rows, where it
    // may take two row blocks only (28672 x 4096: 24.8 against 23.7 us).
    p->decode = false;
    p->skinny = true;
    p->mb = 1;
    R = mid_rows(1);
  }
  // Batch rows 1..4: the gemv kernel (every wave requests a whole round of
  // tiles at once).  Measured on MI355X (Llama-3-8B layers, every bitwidth): four tiles per
  // wave and round; one row block per workgroup at batch 1 and 2 and on layers with few row blocks,
  // two above that (the staged activations of three or four batch rows are then shared); as many
  // waves as there are rounds of four tiles, sixteen at most.  2-bit tiles are half the bytes
  // for the same work per tile: with two row blocks per workgroup (one staging of the
  // activations for both) the 28672 x 4096 layer takes 7.7 instead of 8.4 us; the layers with
  // few row blocks lose that way (4096 x 14336: 6.4 against 5.0 us).
  // Group sizes 32 and -1 run the two shapes named here (a scale per octet, or per row).
  // Five to eight batch rows on layers with few row blocks: there the mid-batch kernel has one
  // workgroup per CU at most and is bound by the instructions it issues per tile; the gemv
  // kernel's instantiation for eight batch rows (two tiles per chain of MFMAs) is ahead up to
  // 512 row blocks - M = 8, 4 bits: 4096 x 14336 9.6 against 11.9 us, 4096 x 4096 4.4 against 5.3,
  // 6144 x 4096 5.5 against 6.0 (two row blocks per workgroup from 320 row blocks on), 8192 x 28672 25.8
  // against 29.5; 2, 3, 6 and 8 bits alike, except 6 bits on 512 row blocks (13.6 against 12.2).  Beyond
  // (10240 x 8192: 16.5 against 14.9; 28672 x 4096: 18.5 against 16.5) the mid-batch kernel's four
  // row blocks per staged activation tile win.
  const bool eight_domain = M > kGemvMaxM && M <= kGemvEightMaxM && group_size != 32;
  const bool eight_auto = eight_domain && variant == 0 &&
                          (row_blocks < 320 || (row_blocks <= 512 && !(bits == 6 && row_blocks > 384)));
  const bool gemv_eight = eight_domain && (variant >= 100 || eight_auto);
  if ((M <= kGemvMaxM || gemv_eight) && flavour == 0 && (variant == 0 || variant >= 100)) {
    // (two batch rows have an instantiation of their own, which stages two rows where the one for
    // three and four stages four: with it one row block per workgroup is ahead at M = 2 as well -
    // 28672 x 4096: 4 bits 11.5 against 12.6 us, 6 bits 16.1 against 17.5, 3 bits 10.7 against 11.5 on the
    // four-row-block shape)
    int shape = ((M >= 3 && row_blocks >= 320) || (bits == 2 && group_size == 128 && row_blocks >= 1024)) ? 2 : 1;
    // three or four batch rows, 2 or 3 bits, many row blocks: four row blocks per workgroup share one
    // staging of the activations and their codes still fit the registers of eight waves
    // per SIMD (28672 x 4096 at M = 4: 3 bits 11.8 against 13.1 us, 2 bits 9.35 against 10.0;
    // 4 bits 14.9 against 13.5: its 64 registers of codes leave four waves per SIMD)
    if (M >= 3 && bits <= 3 && group_size == 128 && row_blocks >= 1024) shape = 6;
    if (M > kGemvMaxM) shape = row_blocks < 320 ? 1 : 2;
    if (variant >= 100) {
      shape = variant - 100;
      if (shape >= kNumGemvShapes) return MATGPTQ_EVARIANT;
      if ((group_size != 128 || M > kGemvMaxM) && shape != 1 && shape != 2) return MATGPTQ_EVARIANT;
    }
    const int T = kGemvShapes[shape][0];
    int Wg = (int)((flags >> MATGPTQ_FLAG_GEMV_WAVES_SHIFT) & 31u);
    const bool waves_given = Wg != 0;
    if (Wg == 0) {
      Wg = (k_tiles + T - 1) / T;
      if (Wg > 16) Wg = 16;
    }
    if (Wg > 16) return MATGPTQ_EVARIANT;
    if (M > kGemvMaxM) {
      // eight batch rows of X' per wave, the table of their sums, the zero block and the wave's
      // partial sums: as many waves as fit the LDS of a CU
      const int per_wave = 8 * (T * 256 + 16) + 256 + 8 * T * 8 + kGemvShapes[shape][1] * 4 * 256;
      const int fit = 160 * 1024 / per_wave;
      if (Wg > fit) {
        if (waves_given) return MATGPTQ_EVARIANT;
        Wg = fit;
      }
    }
    p->gemv = true;
    p->decode = false;
    p->skinny = false;
    p->shape = shape;
    p->R = kGemvShapes[shape][1];
    p->S = 0;
    p->W = Wg;
    p->kc = 0;
    p->stream = false;
    p->smem = 0;
    p->pad = (size_t)((flags >> MATGPTQ_FLAG_GEMV_LDS_SHIFT) & 63u) * 4096u;
    if (p->pad > 160 * 1024) return MATGPTQ_EVARIANT;
    return MATGPTQ_OK;
  }
  if (variant != 0) {
    if (variant >= 100) return MATGPTQ_EVARIANT;
    if (variant >= 91) {  // mid-batch kernel, eight row blocks and 32 batch rows per workgroup
      if (variant > 91 || !eight_rows) return MATGPTQ_EVARIANT;
      p->decode = false;
      p->skinny = true;
      R = 8;
      p->mb = 2;
    } else if (variant >= 89) {  // prefill tiles 16 and up
      p->decode = false;
      p->skinny = false;
      p->cfg = variant - 89 + 16;
    } else if (variant >= 80) {
      p->decode = false;
      p->skinny = true;
      R = 1 << ((variant - 80) % 3);
      p->mb = 1 << ((variant - 80) / 3);
    } else if (variant >= 64) {
      if (variant - 64 > 15) return MATGPTQ_EVARIANT;
      p->decode = false;
      p->skinny = false;
      p->cfg = variant - 64;
    } else {
      if (M > kDecodeMaxM) return MATGPTQ_EVARIANT;
      const int v = variant - 1;
      if (v >= 3 * kNumShapes) return MATGPTQ_EVARIANT;
      p->decode = true;
      p->skinny = false;
      R = 1 << (v % 3);
      S = kShapes[v / 3][0];
      W = kShapes[v / 3][1];
      if (W > k_tiles) return MATGPTQ_EVARIANT;
    }
  }
  if (!p->decode) {
    // the prefill kernel addresses X through a 32-bit buffer offset
    if ((uint64_t)M * (uint64_t)K * 2u >= (1ull << 32)) return MATGPTQ_ESIZE;
    p->R = p->S = p->W = p->kc = 0;
    if (p->skinny) {  // (a forced variant may ask for more than the format takes)
      const int most = eight_rows && p->mb == 2 ? 8 : r_max;
      p->R = R > most ? most : R;
    }
    p->stream = false;
    p->smem = 0;
    return MATGPTQ_OK;
  }
  // burst keeps at most eight waves per workgroup
  const bool stream = flavour == 2 || (flavour == 0 && S * W > 8);
  if (!stream && S * W > 8) return MATGPTQ_EVARIANT;
  // largest kc whose activations fit next to the partial sums and scales
  const int64_t fixed = (int64_t)decode_lds_bytes(R, S, W, 0, 0);
  const int64_t avail = (int64_t)kLdsBudget - fixed;
  int64_t kc = avail > 0 ? (avail / (2 * M) - 8) / 128 : 0;
  if (kc < 1) return variant != 0 ? MATGPTQ_EVARIANT : MATGPTQ_ESIZE;
  if (kc > k_tiles) kc = k_tiles;
  if (kc >= W) kc = kc / W * W;
  p->R = R;
  p->S = S;
  p->W = W;
  p->kc = (int)kc;
  p->stream = stream;
  p->smem = decode_lds_bytes(R, S, W, (int)kc, M);
  if (kc < k_tiles && S * W > 8) return variant != 0 ? MATGPTQ_EVARIANT : MATGPTQ_ESIZE;
  (void)bits;
  return MATGPTQ_OK;
}

// `bf16`: activations, scales, zeros and output are stored as bfloat16 (same kernels built a
// second time with the conversions at their edges)
hipError_t launch_decode(int bits, bool bf16, const GemmArgs& a, int g, const Plan& p, hipStream_t s) {
#define MATGPTQ_CASE(B)                                                                      \
  case B:                                                                                    \
    return bf16 ? launch_decode_b##B##_bf16(a, g, p.R, p.S, p.W, p.kc, p.stream, p.smem, s)  \
                : launch_decode_b##B(a, g, p.R, p.S, p.W, p.kc, p.stream, p.smem, s);
  switch (bits) {
    MATGPTQ_CASE(2)
    MATGPTQ_CASE(3)
    MATGPTQ_CASE(4)
    MATGPTQ_CASE(6)
    default:
      return bf16 ? launch_decode_b8_bf16(a, g, p.R, p.S, p.W, p.kc, p.stream, p.smem, s)
                  : launch_decode_b8(a, g, p.R, p.S, p.W, p.kc, p.stream, p.smem, s);
  }
#undef MATGPTQ_CASE
}

hipError_t launch_prefill(int bits, bool bf16, const GemmArgs& a, int g, const Plan& p, hipStream_t s) {
#define MATGPTQ_CASE(B) \
  case B: return bf16 ? launch_prefill_b##B##_bf16(a, g, p.cfg, s) : launch_prefill_b##B(a, g, p.cfg, s);
  switch (bits) {
    MATGPTQ_CASE(2)
    MATGPTQ_CASE(3)
    MATGPTQ_CASE(4)
    MATGPTQ_CASE(6)
    default: return bf16 ? launch_prefill_b8_bf16(a, g, p.cfg, s) : launch_prefill_b8(a, g, p.cfg, s);
  }
#undef MATGPTQ_CASE
}

// master: `a.packed` holds master-resident bit planes
hipError_t launch_gemv(int bits, bool bf16, const GemmArgs& a, int g, const Plan& p, bool master, hipStream_t s) {
#define MATGPTQ_CASE(B) \
  case B: return bf16 ? launch_gemv_b##B##_bf16(a, g, p.shape, p.W, p.pad, master, s) \
                      : launch_gemv_b##B(a, g, p.shape, p.W, p.pad, master, s);
  switch (bits) {
    MATGPTQ_CASE(2)
    MATGPTQ_CASE(3)
    MATGPTQ_CASE(4)
    MATGPTQ_CASE(6)
    default: return bf16 ? launch_gemv_b8_bf16(a, g, p.shape, p.W, p.pad, master, s)
                         : launch_gemv_b8(a, g, p.shape, p.W, p.pad, master, s);
  }
#undef MATGPTQ_CASE
}

hipError_t launch_skinny(int bits, bool bf16, const GemmArgs& a, int g, const Plan& p, bool master, hipStream_t s) {
#define MATGPTQ_CASE(B) \
  case B: return bf16 ? launch_skinny_b##B##_bf16(a, g, p.R, p.mb, master, s) : launch_skinny_b##B(a, g, p.R, p.mb, master, s);
  switch (bits) {
    MATGPTQ_CASE(2)
    MATGPTQ_CASE(3)
    MATGPTQ_CASE(4)
    MATGPTQ_CASE(6)
    default: return bf16 ? launch_skinny_b8_bf16(a, g, p.R, p.mb, master, s) : launch_skinny_b8(a, g, p.R, p.mb, master, s);
  }
#undef MATGPTQ_CASE
}

}  // namespace
}  // namespace matgptq

using namespace matgptq;

extern "C" {

int matgptq_abi_version(void) { return MATGPTQ_ABI_VERSION; }

const char* matgptq_strerror(int code) {
  switch (code) {
    case MATGPTQ_OK: return "ok";
    case MATGPTQ_EBITS: return "bitwidth must be one of {2, 3, 4, 6, 8}";
    case MATGPTQ_EGROUP: return "group_size must be one of {-1, 32, 128} and divide n_in_features";
    case MATGPTQ_ESHAPE:
      return "n_out_features must be a multiple of 16 and n_in_features a multiple of 128 (or, at group sizes 32 and -1, "
             "such a multiple plus 64; master-resident planes: a multiple of 128)";
    case MATGPTQ_ENULL: return "null pointer argument";
    case MATGPTQ_EDTYPE: return "unsupported data type for this operation (float16 only)";
    case MATGPTQ_ELAUNCH: return "HIP launch failed";
    case MATGPTQ_EVARIANT: return "forced kernel variant does not apply to this problem";
    case MATGPTQ_ESIZE: return "size exceeds the supported maximum";
    case MATGPTQ_EWORKSPACE: return "workspace missing or smaller than matgptq_gemm_master_workspace_bytes()";
    case MATGPTQ_EALIAS: return "an output buffer overlaps an input that other workgroups still read";
    case MATGPTQ_ESTATIC:
      return "the sliced tensor is larger than the library's built-in workspace (MATGPTQ_STATIC_WORKSPACE_BYTES): "
             "use matgptq_gemm_master with a workspace";
    default: return "unknown error";
  }
}

// The kernels that read master-resident bit planes themselves: the gemv kernel in its two shapes
// built for them, and the mid-batch kernel.
// (the gemv kernel reads the planes in every batch size it is planned for: one to four rows, and five
// to eight with one scale per tile or row)
static bool plan_reads_planes(const Plan& p, int64_t M) {
  return (p.gemv && M <= kGemvEightMaxM && (p.shape == 1 || p.shape == 2)) || p.skinny;
}

// checks, plan, launch; `master_planes`: the weight operand is master-resident bit planes and
// the plan must be one of those kernels (the caller has made sure of it)
static int run_gemm(int bitwidth, int group_size, int64_t N, int64_t K, int64_t M, const void* weights_dev,
                    const void* scales_dev, const void* zeros_dev, const void* x_dev, void* y_dev,
                    void* stream, uint32_t flags, bool master_planes) {
  if (int e = check_problem(bitwidth, group_size, N, K)) return e;
  if (M <= 0 || M > (1 << 24) || N > (1 << 24) || K > (1 << 24)) return MATGPTQ_ESIZE;
  // the kernels address the weight tensor with 32-bit byte offsets
  if ((uint64_t)N * (uint64_t)K / 8 * (uint64_t)(master_planes ? 8 : bitwidth) >= (1ull << 32)) return MATGPTQ_ESIZE;
  if (!weights_dev || !scales_dev || !x_dev || !y_dev) return MATGPTQ_ENULL;
  Plan p;
  if (int e = make_plan(bitwidth, group_size, N, K, M, zeros_dev != nullptr, flags, &p)) return e;
  if (master_planes && !plan_reads_planes(p, M)) return MATGPTQ_EVARIANT;
  GemmArgs a;
  a.packed = static_cast<const uint32_t*>(weights_dev);
  a.scales = static_cast<const uint16_t*>(scales_dev);
  a.zeros = static_cast<const uint16_t*>(zeros_dev);
  a.x = static_cast<const uint16_t*>(x_dev);
  a.y = static_cast<uint16_t*>(y_dev);
  a.N = (int)N;
  a.K = (int)K;
  a.M = (int)M;
  a.G = group_size == -1 ? 1 : (int)(K / group_size);
  a.k_tiles = (int)(K / 128);
  a.row_blocks = (int)(N / 16);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool bf16 = (flags & MATGPTQ_FLAG_BF16) != 0;
  const hipError_t err = p.gemv     ? launch_gemv(bitwidth, bf16, a, group_size, p, master_planes, s)
                         : p.decode ? launch_decode(bitwidth, bf16, a, group_size, p, s)
                         : p.skinny ? launch_skinny(bitwidth, bf16, a, group_size, p, master_planes, s)
                                    : launch_prefill(bitwidth, bf16, a, group_size, p, s);
  if (err != hipSuccess) return MATGPTQ_ELAUNCH;
  // K = 128 t + 64: the kernels above have multiplied the t tiles; a second launch adds the last 64 columns
  if (K % 128 != 0 && launch_tail_gemm(bitwidth, bf16, a, group_size, s) != hipSuccess) return MATGPTQ_ELAUNCH;
  if (!(flags & MATGPTQ_FLAG_ASYNC)) {
    if (hipStreamSynchronize(s) != hipSuccess) return MATGPTQ_ELAUNCH;
  }
  return MATGPTQ_OK;
}

int matgptq_gemm(int bitwidth, int group_size, int64_t N, int64_t K, int64_t M,
                 const void* packed_dev, const void* scales_dev, const void* zeros_dev,
                 const void* x_dev, void* y_dev, void* stream, uint32_t flags) {
  return run_gemm(bitwidth, group_size, N, K, M, packed_dev, scales_dev, zeros_dev, x_dev, y_dev, stream,
                  flags, false);
}

int matgptq_gemm_prologue(int bitwidth, int group_size, int64_t N, int64_t K, int64_t M,
                          const void* packed_dev, const void* scales_dev, const void* zeros_dev,
                          int kind, const void* a_dev, const void* b_dev, const void* w_dev, void* out_dev,
                          float eps, void* y_dev, void* stream, uint32_t flags) {
  if (int e = check_problem(bitwidth, group_size, N, K)) return e;
  if (M <= 0) return MATGPTQ_ESIZE;
  if ((uint64_t)N * (uint64_t)K / 8 * (uint64_t)bitwidth >= (1ull << 32)) return MATGPTQ_ESIZE;
  if (!packed_dev || !scales_dev || !a_dev || !y_dev) return MATGPTQ_ENULL;
  if (kind != MATGPTQ_PRE_SILU_MUL && kind != MATGPTQ_PRE_ADD_RMSNORM) return MATGPTQ_EVARIANT;
  if (group_size != 128 || (flags & MATGPTQ_FLAG_BF16) || M > kGemvMaxM || K % 128 != 0) return MATGPTQ_EVARIANT;
  if (flags & (MATGPTQ_FLAG_VARIANT_MASK | MATGPTQ_FLAG_FLAVOUR_MASK)) return MATGPTQ_EVARIANT;
  const int k_tiles = (int)(K / 128);
  if (kind == MATGPTQ_PRE_ADD_RMSNORM) {
    if (!w_dev) return MATGPTQ_ENULL;
    if (k_tiles > 64) return MATGPTQ_EVARIANT;  // the mean needs all of K inside one round of a workgroup
    const size_t row_bytes = (size_t)M * (size_t)K * 2;
    auto overlaps = [&](const void* p) {
      const char *o = static_cast<const char*>(out_dev), *q = static_cast<const char*>(p);
      return p != nullptr && o < q + row_bytes && q < o + row_bytes;
    };
    if (out_dev && (overlaps(a_dev) || overlaps(b_dev))) return MATGPTQ_EALIAS;
  }
  Plan p;
  if (int e = make_plan(bitwidth, group_size, N, K, M, zeros_dev != nullptr, flags, &p)) return e;
  if (!p.gemv) return MATGPTQ_EVARIANT;
  // the two shapes built with prologues: four tiles per wave, one or two row blocks per workgroup
  const int shape = p.R >= 2 ? 2 : 1;
  int W = (k_tiles + 3) / 4;
  if (W > 16) W = 16;
  GemmArgs a;
  a.packed = static_cast<const uint32_t*>(packed_dev);
  a.scales = static_cast<const uint16_t*>(scales_dev);
  a.zeros = static_cast<const uint16_t*>(zeros_dev);
  a.x = static_cast<const uint16_t*>(a_dev);
  a.y = static_cast<uint16_t*>(y_dev);
  a.N = (int)N;
  a.K = (int)K;
  a.M = (int)M;
  a.G = (int)(K / group_size);
  a.k_tiles = k_tiles;
  a.row_blocks = (int)(N / 16);
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipError_t err;
  switch (bitwidth) {
    case 2: err = launch_gemv_prologue_b2(a, kind, shape, W, b_dev, w_dev, out_dev, eps, s); break;
    case 3: err = launch_gemv_prologue_b3(a, kind, shape, W, b_dev, w_dev, out_dev, eps, s); break;
    case 4: err = launch_gemv_prologue_b4(a, kind, shape, W, b_dev, w_dev, out_dev, eps, s); break;
    case 6: err = launch_gemv_prologue_b6(a, kind, shape, W, b_dev, w_dev, out_dev, eps, s); break;
    default: err = launch_gemv_prologue_b8(a, kind, shape, W, b_dev, w_dev, out_dev, eps, s); break;
  }
  if (err != hipSuccess) return MATGPTQ_ELAUNCH;
  if (!(flags & MATGPTQ_FLAG_ASYNC) && hipStreamSynchronize(s) != hipSuccess) return MATGPTQ_ELAUNCH;
  return MATGPTQ_OK;
}

// does the GEMM at this shape read the planes itself (gemv and mid-batch kernels), or does it need
// the pre-sliced tensor in a workspace first?
// `flags` comes back with the plan to take: up to 128 batch rows a shape whose own plan needs the
// workspace is given the mid-batch kernel instead (its largest shape for that batch size), which
// costs 1.05 .. 1.4 times its time on pre-sliced codes but saves the slicing pass - 41 us for the
// 117 M codes of a 28672 x 4096 layer, more than such a product takes.
static int master_reads_planes(int bitwidth, int group_size, int64_t N, int64_t K, int64_t M, bool zp,
                               uint32_t* flags, bool* direct) {
  if (int e = check_problem(bitwidth, group_size, N, K)) return e;
  if (K % 128 != 0) return MATGPTQ_ESHAPE;  // the bit planes have whole tiles only
  if (M <= 0) return MATGPTQ_ESIZE;
  Plan p;
  if (int e = make_plan(bitwidth, group_size, N, K, M, zp, *flags, &p)) return e;
  *direct = plan_reads_planes(p, M);
  const bool automatic = (*flags & MATGPTQ_FLAG_VARIANT_MASK) == 0 && ((*flags >> 16) & 3u) == 0;
  if (!*direct && automatic && M <= kGemvMaxM) {
    // the planner's own gemv shape for this problem has no instantiation on planes (four row blocks
    // per workgroup at 2 and 3 bits): the two-row-block shape, which has one, serves every batch of
    // one to four rows
    const uint32_t forced = *flags | ((100u + 2u) << MATGPTQ_FLAG_VARIANT_SHIFT);
    if (make_plan(bitwidth, group_size, N, K, M, zp, forced, &p) == MATGPTQ_OK && plan_reads_planes(p, M)) {
      *flags = forced;
      *direct = true;
    }
  }
  if (!*direct && automatic && M > kGemvMaxM && M <= 128) {
    const uint32_t msel = M <= 16 ? 0u : M <= 32 ? 1u : 2u;  // 16, 32 or 64 batch rows per workgroup
    const uint32_t forced = *flags | ((80u + 2u + 3u * msel) << MATGPTQ_FLAG_VARIANT_SHIFT);  // four row blocks, or as many as fit
    if (make_plan(bitwidth, group_size, N, K, M, zp, forced, &p) == MATGPTQ_OK && plan_reads_planes(p, M)) {
      *flags = forced;
      *direct = true;
    }
  }
  return MATGPTQ_OK;
}

size_t matgptq_gemm_master_workspace_bytes(int bitwidth, int group_size, int64_t N, int64_t K, int64_t M,
                                           uint32_t flags) {
  // The plan can depend on whether the call brings zero points: the workspace covers both forms, so
  // that a size asked for once per layer holds for either call.
  for (int zp = 0; zp < 2; ++zp) {
    bool direct = false;
    uint32_t f = flags;
    if (master_reads_planes(bitwidth, group_size, N, K, M, zp != 0, &f, &direct) != MATGPTQ_OK) return 0;
    if (!direct) return matgptq_packed_words(bitwidth, N, K) * 4;
  }
  return 0;
}

static int gemm_master_impl(int bitwidth, int group_size, int64_t N, int64_t K, int64_t M,
                            const void* planes_dev, const void* scales_dev, const void* zeros_dev,
                            const void* x_dev, void* y_dev, void* workspace_dev, size_t workspace_bytes,
                            void* stream, uint32_t flags) {
  bool direct = false;
  if (int e = master_reads_planes(bitwidth, group_size, N, K, M, zeros_dev != nullptr, &flags, &direct)) return e;
  if (!planes_dev) return MATGPTQ_ENULL;
  if (direct)
    return run_gemm(bitwidth, group_size, N, K, M, planes_dev, scales_dev, zeros_dev, x_dev, y_dev, stream,
                    flags, true);
  // two launches: slice the planes into the pre-sliced layout, then the GEMM of that regime
  const size_t need = matgptq_packed_words(bitwidth, N, K) * 4;
  if (!workspace_dev || workspace_bytes < need) return MATGPTQ_EWORKSPACE;
  if (launch_master_slice(static_cast<const uint32_t*>(planes_dev), N, K, bitwidth, true, workspace_dev,
                          static_cast<hipStream_t>(stream)) != hipSuccess)
    return MATGPTQ_ELAUNCH;
  return run_gemm(bitwidth, group_size, N, K, M, workspace_dev, scales_dev, zeros_dev, x_dev, y_dev, stream,
                  flags, false);
}

int matgptq_gemm_master(int bitwidth, int group_size, int64_t N, int64_t K, int64_t M,
                        const void* planes_dev, const void* scales_dev, const void* zeros_dev,
                        const void* x_dev, void* y_dev, void* workspace_dev, size_t workspace_bytes,
                        void* stream, uint32_t flags) {
  return gemm_master_impl(bitwidth, group_size, N, K, M, planes_dev, scales_dev, zeros_dev, x_dev, y_dev,
                          workspace_dev, workspace_bytes, stream, flags);
}

// Address of this GPU's copy of `scratch`: looked up once per device, with that device current
// (the array's name is only a host-side handle, not a device address).
// The current device has to be the one that owns the call's stream (as for every entry point here:
// the kernels are launched on the current device's copy of the code object).
static int static_scratch(void** ptr) {
  constexpr int kMaxDevices = 64;
  static std::mutex lock;
  static void* addr[kMaxDevices] = {};
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return MATGPTQ_ELAUNCH;
  std::lock_guard<std::mutex> guard(lock);
  if (addr[dev] == nullptr) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) return MATGPTQ_ELAUNCH;
    addr[dev] = p;
  }
  *ptr = addr[dev];
  return MATGPTQ_OK;
}

int matgptq_gemm_master_static(int bitwidth, int group_size, int64_t N, int64_t K, int64_t M,
                               const void* planes_dev, const void* scales_dev, const void* zeros_dev,
                               const void* x_dev, void* y_dev, void* stream, uint32_t flags) {
  bool direct = false;
  uint32_t plan_flags = flags;  // (gemm_master_impl decides again from the caller's flags, the same way)
  if (int e = master_reads_planes(bitwidth, group_size, N, K, M, zeros_dev != nullptr, &plan_flags, &direct)) return e;
  void* ws = nullptr;
  size_t need = 0;
  if (!direct) {
    need = matgptq_packed_words(bitwidth, N, K) * 4;
    if (need > kStaticScratchBytes) return MATGPTQ_ESTATIC;
    if (int e = static_scratch(&ws)) return e;
  }
  return gemm_master_impl(bitwidth, group_size, N, K, M, planes_dev, scales_dev, zeros_dev, x_dev, y_dev, ws,
                          need, stream, flags);
}

int matgptq_pack_master_device(const uint8_t* codes_dev, int64_t N, int64_t K, uint32_t* planes_dev,
                               void* stream) {
  if (int e = check_problem(8, -1, N, K)) return e;
  if (K % 128 != 0) return MATGPTQ_ESHAPE;
  if (!codes_dev || !planes_dev) return MATGPTQ_ENULL;
  return launch_pack_master(codes_dev, N, K, planes_dev, static_cast<hipStream_t>(stream)) == hipSuccess
             ? MATGPTQ_OK : MATGPTQ_ELAUNCH;
}

int matgptq_unpack_master_device(const uint32_t* planes_dev, int64_t N, int64_t K, int bitwidth,
                                 uint8_t* codes_dev, void* stream) {
  if (int e = check_problem(bitwidth, -1, N, K)) return e;
  if (K % 128 != 0) return MATGPTQ_ESHAPE;
  if (!planes_dev || !codes_dev) return MATGPTQ_ENULL;
  return launch_master_slice(planes_dev, N, K, bitwidth, false, codes_dev, static_cast<hipStream_t>(stream)) ==
                 hipSuccess ? MATGPTQ_OK : MATGPTQ_ELAUNCH;
}

int matgptq_probe_read(const void* buf_dev, size_t bytes, void* stream) {
  if (!buf_dev) return MATGPTQ_ENULL;
  if (bytes == 0 || bytes % 16 != 0) return MATGPTQ_ESIZE;
  return launch_read_probe(buf_dev, bytes, static_cast<hipStream_t>(stream)) == hipSuccess ? MATGPTQ_OK
                                                                                          : MATGPTQ_ELAUNCH;
}

int matgptq_describe_plan(int bitwidth, int group_size, int64_t N, int64_t K, int64_t M,
                          int has_zeros, uint32_t flags, char* buf, size_t buf_len) {
  if (int e = check_problem(bitwidth, group_size, N, K)) return e;
  if (!buf || buf_len == 0) return MATGPTQ_ENULL;
  if (M <= 0) return MATGPTQ_ESIZE;
  Plan p;
  if (int e = make_plan(bitwidth, group_size, N, K, M, has_zeros != 0, flags, &p)) return e;
  if (p.gemv)
    snprintf(buf, buf_len, "gemv b%d g%d zp%d T%d R%d W%d pad%zu", bitwidth, group_size, has_zeros ? 1 : 0,
             kGemvShapes[p.shape][0], p.R, p.W, p.pad);
  else if (p.decode)
    snprintf(buf, buf_len, "decode-%s b%d g%d zp%d R%d S%d W%d kc%d lds%zu",
             p.kc < (int)(K / 128) ? "chunked" : (p.stream ? "stream" : "burst"), bitwidth, group_size,
             has_zeros ? 1 : 0, p.R, p.S, p.W, p.kc, p.smem);
  else if (p.skinny)
    snprintf(buf, buf_len, "midbatch b%d g%d zp%d R%d mb%d", bitwidth, group_size, has_zeros ? 1 : 0,
             p.R, p.mb);
  else
    snprintf(buf, buf_len, "prefill b%d g%d zp%d cfg%d", bitwidth, group_size, has_zeros ? 1 : 0,
             p.cfg);
  return MATGPTQ_OK;
}

int matgptq_pack_device(const uint8_t* codes_dev, int64_t N, int64_t K, int bitwidth,
                        int slice_from_master, uint32_t* out_dev, void* stream) {
  if (int e = check_problem(bitwidth, -1, N, K)) return e;
  if (!codes_dev || !out_dev) return MATGPTQ_ENULL;
  return launch_pack(codes_dev, N, K, bitwidth, slice_from_master, out_dev,
                     static_cast<hipStream_t>(stream)) == hipSuccess ? MATGPTQ_OK : MATGPTQ_ELAUNCH;
}

int matgptq_unpack_device(const uint32_t* packed_dev, int64_t N, int64_t K, int bitwidth,
                          uint8_t* codes_dev, void* stream) {
  if (int e = check_problem(bitwidth, -1, N, K)) return e;
  if (!packed_dev || !codes_dev) return MATGPTQ_ENULL;
  return launch_unpack(packed_dev, N, K, bitwidth, codes_dev, static_cast<hipStream_t>(stream)) ==
                 hipSuccess ? MATGPTQ_OK : MATGPTQ_ELAUNCH;
}

int matgptq_reorder_scales_device(const uint16_t* in_dev, int64_t N, int64_t K, int group_size,
                                  uint16_t* out_dev, void* stream) {
  if (int e = check_problem(8, group_size, N, K)) return e;
  if (!in_dev || !out_dev) return MATGPTQ_ENULL;
  const int64_t G = group_size == -1 ? 1 : K / group_size;
  return launch_reorder(in_dev, N, G, out_dev, static_cast<hipStream_t>(stream)) == hipSuccess
             ? MATGPTQ_OK : MATGPTQ_ELAUNCH;
}

int matgptq_slice_device(const uint8_t* master_dev, int64_t count, int bitwidth,
                         uint8_t* sliced_dev, void* stream) {
  if (!valid_bits(bitwidth)) return MATGPTQ_EBITS;
  if (count < 0) return MATGPTQ_ESIZE;
  if (count == 0) return MATGPTQ_OK;
  if (!master_dev || !sliced_dev) return MATGPTQ_ENULL;
  return launch_slice(master_dev, count, bitwidth, sliced_dev, static_cast<hipStream_t>(stream)) ==
                 hipSuccess ? MATGPTQ_OK : MATGPTQ_ELAUNCH;
}

int matgptq_dequantize_device(int bitwidth, int group_size, int64_t N, int64_t K,
                              const void* packed_dev, const void* scales_dev,
                              const void* zeros_dev, void* w_dev, void* stream) {
  if (int e = check_problem(bitwidth, group_size, N, K)) return e;
  if (!packed_dev || !scales_dev || !w_dev) return MATGPTQ_ENULL;
  return launch_dequant(bitwidth, group_size, N, K, static_cast<const uint32_t*>(packed_dev),
                        static_cast<const uint16_t*>(scales_dev),
                        static_cast<const uint16_t*>(zeros_dev), static_cast<uint16_t*>(w_dev),
                        static_cast<hipStream_t>(stream)) == hipSuccess ? MATGPTQ_OK : MATGPTQ_ELAUNCH;
}

}  // extern "C"
