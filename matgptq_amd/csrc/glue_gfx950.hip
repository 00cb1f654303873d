// The operators between the bit-sliced linears of a decoder block at decode time, fused so that
// a block is nine launches: residual add + RMS norm, rotary embedding + cache write, attention
// of a few query rows over a static key/value cache, SiLU gate.  They belong to the end-to-end
// decode measurement (the reference leaves these operators to transformers / vLLM,
// inference_lib/inference_demo_transformers.py:134-176, inference_lib/bench_transformers_e2e.py:61-76)
// and are built into a library of their own, apart from the GEMM's C ABI.  fp16 storage, fp32
// arithmetic.  All of them are small and latency-bound: one workgroup per row / head.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "../../include/matgptq_glue.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));

constexpr int kThreads = 256;

int launch_status() { return hipGetLastError() == hipSuccess ? 0 : MATGPTQ_GLUE_ELAUNCH; }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
// sum over the 256 threads of a workgroup; `red` holds 4 floats and is reused, so the
// leading barrier keeps a later call from overwriting values an earlier one is still reading
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return red[0] + red[1] + red[2] + red[3];
}
// h += delta (if given); x = h * rsqrt(mean(h^2) + eps) * weight.  One workgroup per row; a thread
// keeps its chunks of the row in registers (H <= 8 * 256 * kMaxChunks).
constexpr int kMaxChunks = 4;
__global__ void __launch_bounds__(kThreads)
add_rmsnorm_kernel(_Float16* __restrict__ h, const _Float16* __restrict__ delta,
                   const _Float16* __restrict__ weight, _Float16* __restrict__ x, int H, float eps) {
  __shared__ float red[4];
  const int chunks = H / 8;
  half8* hr = reinterpret_cast<half8*>(h + (size_t)blockIdx.x * H);
  const half8* dr = delta ? reinterpret_cast<const half8*>(delta + (size_t)blockIdx.x * H) : nullptr;
  const half8* wr = reinterpret_cast<const half8*>(weight);
  half8 v[kMaxChunks], w[kMaxChunks];
  float ss = 0.f;
  // (the weights are requested together with the row: one round trip to memory, not two)
#pragma unroll
  for (int i = 0; i < kMaxChunks; i++) {
    const int c = threadIdx.x + i * kThreads;
    if (c < chunks) w[i] = wr[c];
  }
#pragma unroll
  for (int i = 0; i < kMaxChunks; i++) {
    const int c = threadIdx.x + i * kThreads;
    if (c < chunks) {
      v[i] = hr[c];
      if (dr) {
        v[i] = v[i] + dr[c];  // one fp16 rounding, like the residual add it replaces
        hr[c] = v[i];
      }
#pragma unroll
      for (int e = 0; e < 8; e++) ss += (float)v[i][e] * (float)v[i][e];
    }
  }
  const float rs = rsqrtf(block_sum(ss, red) / (float)H + eps);
  half8* xr = reinterpret_cast<half8*>(x + (size_t)blockIdx.x * H);
#pragma unroll
  for (int i = 0; i < kMaxChunks; i++) {
    const int c = threadIdx.x + i * kThreads;
    if (c < chunks) {
      half8 o;
#pragma unroll
      for (int e = 0; e < 8; e++) o[e] = (_Float16)((float)v[i][e] * rs * (float)w[i][e]);
      xr[c] = o;
    }
  }
}

// One element of the rotary embedding: own * cos + other * sin, where `other` is the partner of
// the half-split pair with its sign (minus the upper partner for the lower half, plus the lower
// partner for the upper half).  One expression for every kernel, so that all of them round alike.
__device__ __forceinline__ _Float16 rotary(float own, float other, _Float16 c, _Float16 s) {
  return (_Float16)(own * (float)c + other * (float)s);
}

// Rotary embedding (half-split pairs) of the query and key heads of one row of the fused qkv
// output; queries are rotated in place, rotated keys and the values go to row pos[m] of the
// caches [kv_heads, max_ctx, d].  Grid (heads + 2 kv_heads, M), 64 threads.
__global__ void __launch_bounds__(64)
rope_cache_kernel(_Float16* __restrict__ qkv, const _Float16* __restrict__ cos_t,
                  const _Float16* __restrict__ sin_t, const int64_t* __restrict__ pos,
                  _Float16* __restrict__ k_cache, _Float16* __restrict__ v_cache, int heads, int kv_heads,
                  int d, int64_t max_ctx) {
  const int head = blockIdx.x, m = blockIdx.y;
  int64_t p = pos[m];
  p = p < 0 ? 0 : (p >= max_ctx ? max_ctx - 1 : p);  // never outside the tables and caches
  _Float16* src = qkv + ((size_t)m * (heads + 2 * kv_heads) + head) * d;
  if (head >= heads + kv_heads) {
    _Float16* dst = v_cache + ((size_t)(head - heads - kv_heads) * max_ctx + p) * d;
    for (int i = threadIdx.x; i < d; i += 64) dst[i] = src[i];
    return;
  }
  _Float16* dst = head < heads ? src : k_cache + ((size_t)(head - heads) * max_ctx + p) * d;
  const _Float16* c = cos_t + (size_t)p * d;
  const _Float16* s = sin_t + (size_t)p * d;
  const int half = d / 2;
  for (int i = threadIdx.x; i < half; i += 64) {
    const float a = (float)src[i], b = (float)src[i + half];
    dst[i] = rotary(a, -b, c[i], s[i]);
    dst[i + half] = rotary(b, a, c[i + half], s[i + half]);
  }
}

// Attention of one query head of one row over the cache positions 0 .. pos[m] (head dimension
// 128).  The kernel is bound by the latency of its cache reads, not by their volume, so it runs
// wide: 1024 threads, sixteen lanes share a cache row (16 bytes each), 64 rows per step of the
// workgroup and eight steps in flight per thread.  The scores wait in LDS for the softmax, then
// the same walk accumulates the values.
// Grid (heads, M), dynamic LDS: max_ctx floats + 16 x 128 floats + 16.
constexpr int kAttnThreads = 1024;
constexpr int kAttnWaves = kAttnThreads / 64;
constexpr int kAttnRows = kAttnThreads / 16;  // cache rows per step
constexpr int kAttnDepth = 8;                 // steps in flight

__device__ __forceinline__ float attn_block_reduce(float v, float* red, bool is_max) {
  v = is_max ? wave_max(v) : wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = red[0];
#pragma unroll
  for (int w = 1; w < kAttnWaves; w++) r = is_max ? fmaxf(r, red[w]) : r + red[w];
  return r;
}

// ROPE (one query row only): the rotary embedding and the cache write of the row happen here as
// well, which saves a launch per block.  The query head is rotated in registers; the row's own
// key (rotated) and value come from qkv instead of the cache, and the workgroup of the first
// query head of each key/value head writes them to the caches for the steps to come (another
// workgroup may read that cache row meanwhile: it does not use what it read).
template <bool ROPE>
__global__ void __launch_bounds__(kAttnThreads)
attention_kernel(const _Float16* __restrict__ qkv, _Float16* k_cache, _Float16* v_cache,
                 const int64_t* __restrict__ pos, _Float16* __restrict__ out,
                 const _Float16* __restrict__ cos_t, const _Float16* __restrict__ sin_t, int heads,
                 int kv_heads, int64_t max_ctx, float scale) {
  extern __shared__ __align__(16) float lds[];
  constexpr int d = 128;
  float* scores = lds;                  // [max_ctx]
  float* part = lds + max_ctx;          // [kAttnWaves][128]
  float* red = part + kAttnWaves * d;   // [kAttnWaves]
  const int head = blockIdx.x, m = blockIdx.y;
  const int kvh = head / (heads / kv_heads);
  int64_t p = pos[m];
  p = p < 0 ? 0 : (p >= max_ctx ? max_ctx - 1 : p);
  const int n = (int)p + 1;
  const int sub = threadIdx.x & 15, grp = threadIdx.x >> 4;

  const _Float16* row = qkv + (size_t)m * (heads + 2 * kv_heads) * d + sub * 8;
  half8 qv = *reinterpret_cast<const half8*>(row + (size_t)head * d);
  half8 k_cur = qv, v_cur = qv;
  if constexpr (ROPE) {
    k_cur = *reinterpret_cast<const half8*>(row + (size_t)(heads + kvh) * d);
    v_cur = *reinterpret_cast<const half8*>(row + (size_t)(heads + kv_heads + kvh) * d);
  }
  const _Float16* kb = k_cache + (size_t)kvh * max_ctx * d + sub * 8;
  const _Float16* vb = v_cache + (size_t)kvh * max_ctx * d + sub * 8;

  // Every load is unconditional and its address does not wait for pos[m]: a row beyond n is
  // read from inside the cache (beyond the cache: its last row) and never used.
  const int last = (int)max_ctx - 1;
  auto row_of = [&](int t) { return (size_t)(t < last ? t : last) * d; };
  // The value rows of the first trip do not depend on the scores: they are requested together
  // with the key rows, so that a context of up to 64 x kAttnDepth rows costs one round trip to
  // memory instead of two.
  half8 v_first[kAttnDepth], k_first[kAttnDepth];
#pragma unroll
  for (int u = 0; u < kAttnDepth; u++) k_first[u] = *reinterpret_cast<const half8*>(kb + row_of(grp + u * kAttnRows));
#pragma unroll
  for (int u = 0; u < kAttnDepth; u++) v_first[u] = *reinterpret_cast<const half8*>(vb + row_of(grp + u * kAttnRows));
  if constexpr (ROPE) {
    // lanes sub and sub ^ 8 of a row group hold the two halves of the rotary pairs
    const half8 cv = *reinterpret_cast<const half8*>(cos_t + (size_t)p * d + sub * 8);
    const half8 sv = *reinterpret_cast<const half8*>(sin_t + (size_t)p * d + sub * 8);
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const float qo = (float)qv[e], ko = (float)k_cur[e];
      const float qp = __shfl_xor(qo, 8, 64), kp = __shfl_xor(ko, 8, 64);
      qv[e] = rotary(qo, sub < 8 ? -qp : qp, cv[e], sv[e]);
      k_cur[e] = rotary(ko, sub < 8 ? -kp : kp, cv[e], sv[e]);
    }
    if (head % (heads / kv_heads) == 0 && grp == 0) {
      *reinterpret_cast<half8*>(k_cache + ((size_t)kvh * max_ctx + p) * d + sub * 8) = k_cur;
      *reinterpret_cast<half8*>(v_cache + ((size_t)kvh * max_ctx + p) * d + sub * 8) = v_cur;
    }
  }
  float q[8];
#pragma unroll
  for (int e = 0; e < 8; e++) q[e] = (float)qv[e] * scale;
  float mx = -INFINITY;
  auto score_trip = [&](int t0, const half8 (&kv)[kAttnDepth]) {
#pragma unroll
    for (int u = 0; u < kAttnDepth; u++) {
      const int t = t0 + u * kAttnRows;
      const half8 kk = ROPE && t == (int)p ? k_cur : kv[u];
      float dot = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e++) dot += q[e] * (float)kk[e];
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) dot += __shfl_xor(dot, o, 64);  // the 16 lanes of a row are adjacent
      if (t < n) {
        if (sub == 0) scores[t] = dot;
        mx = fmaxf(mx, dot);
      }
    }
  };
  // first trip, by every row group whatever n is (its rows were requested above, before
  // anything waited for pos[m])
  score_trip(grp, k_first);
  for (int t0 = grp + kAttnRows * kAttnDepth; t0 < n; t0 += kAttnRows * kAttnDepth) {
    half8 kv[kAttnDepth];
#pragma unroll
    for (int u = 0; u < kAttnDepth; u++) kv[u] = *reinterpret_cast<const half8*>(kb + row_of(t0 + u * kAttnRows));
    score_trip(t0, kv);
  }
  mx = attn_block_reduce(mx, red, true);  // (its barriers also publish the scores)
  float sum = 0.f;
  for (int t = threadIdx.x; t < n; t += kAttnThreads) {
    const float e = __expf(scores[t] - mx);
    scores[t] = e;
    sum += e;
  }
  sum = attn_block_reduce(sum, red, false);

  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int t0 = grp; t0 < n; t0 += kAttnRows * kAttnDepth) {
    half8 vv[kAttnDepth];
    float pr[kAttnDepth];
#pragma unroll
    for (int u = 0; u < kAttnDepth; u++) {
      const int t = t0 + u * kAttnRows;
      vv[u] = t0 == grp ? v_first[u] : *reinterpret_cast<const half8*>(vb + row_of(t));
      if (ROPE && t == (int)p) vv[u] = v_cur;
      pr[u] = t < n ? scores[t] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < kAttnDepth; u++) {
      if (t0 + u * kAttnRows < n) {  // (an unused row may hold anything, also NaN)
#pragma unroll
        for (int e = 0; e < 8; e++) acc[e] += pr[u] * (float)vv[u][e];
      }
    }
  }
  // the four rows of a wave first, then the sixteen waves through LDS
#pragma unroll
  for (int e = 0; e < 8; e++) {
    acc[e] += __shfl_xor(acc[e], 16, 64);
    acc[e] += __shfl_xor(acc[e], 32, 64);
  }
  if ((threadIdx.x & 63) < 16) {
#pragma unroll
    for (int e = 0; e < 8; e++) part[(threadIdx.x >> 6) * d + sub * 8 + e] = acc[e];
  }
  __syncthreads();
  if (threadIdx.x < d) {
    float o = 0.f;
#pragma unroll
    for (int w = 0; w < kAttnWaves; w++) o += part[w * d + threadIdx.x];
    out[((size_t)m * heads + head) * d + threadIdx.x] = (_Float16)(o / sum);
  }
}

// The same attention with the context split over workgroups: grid (kv_heads, splits, M), one
// workgroup per key/value head and 64 cache rows, which serves all REP query heads of that
// key/value head from one read of the rows (a workgroup per query head reads them REP times, and
// a single CU can pull only so much).  Every workgroup with rows to look at leaves its partial
// result - the maximum score, the sum of the exponentials and the weighted values, per query
// head - in `ws`; attention_combine_kernel, launched behind it, puts the partial results of the
// splits up to pos[m] together.  (One kernel whose last workgroup combines was measured slower:
// the fences that publish the partial results across the L2 caches of the XCDs cost more than
// the second launch.)
// ws: M x heads x splits x 130 floats.
constexpr int kSplitRows = 64;
constexpr int kSplitStride = 130;  // 128 values, maximum, sum

template <bool ROPE, int REP>
__global__ void __launch_bounds__(256)
attention_split_kernel(const _Float16* __restrict__ qkv, _Float16* k_cache, _Float16* v_cache,
                       const int64_t* __restrict__ pos, _Float16* __restrict__ out,
                       const _Float16* __restrict__ cos_t, const _Float16* __restrict__ sin_t,
                       float* __restrict__ ws, int heads, int kv_heads, int64_t max_ctx, int splits, float scale) {
  constexpr int d = 128;
  __shared__ float sc[REP][kSplitRows];  // scores, then exponentials
  __shared__ float part[4][REP][d];      // weighted values per wave
  __shared__ float mx_s[REP], sum_s[REP];
  const int kvh = blockIdx.x, split = blockIdx.y, m = blockIdx.z;
  const int tid = threadIdx.x, sub = tid & 15, grp = tid >> 4, wave = tid >> 6, lane = tid & 63;
  const int row0 = split * kSplitRows;
  const int last = (int)max_ctx - 1;
  auto row_of = [&](int t) { return (size_t)(t < last ? t : last) * d; };
  const _Float16* kb = k_cache + (size_t)kvh * max_ctx * d + sub * 8;
  const _Float16* vb = v_cache + (size_t)kvh * max_ctx * d + sub * 8;
  // this thread's rows: row0 + grp + 16 u; requested before anything waits for pos[m]
  half8 kr[4], vr[4];
#pragma unroll
  for (int u = 0; u < 4; u++) kr[u] = *reinterpret_cast<const half8*>(kb + row_of(row0 + grp + 16 * u));
#pragma unroll
  for (int u = 0; u < 4; u++) vr[u] = *reinterpret_cast<const half8*>(vb + row_of(row0 + grp + 16 * u));
  const _Float16* row = qkv + (size_t)m * (heads + 2 * kv_heads) * d + sub * 8;
  half8 qv[REP];
#pragma unroll
  for (int r = 0; r < REP; r++) qv[r] = *reinterpret_cast<const half8*>(row + (size_t)(kvh * REP + r) * d);
  half8 k_cur = qv[0], v_cur = qv[0];
  if constexpr (ROPE) {
    k_cur = *reinterpret_cast<const half8*>(row + (size_t)(heads + kvh) * d);
    v_cur = *reinterpret_cast<const half8*>(row + (size_t)(heads + kv_heads + kvh) * d);
  }
  int64_t p = pos[m];
  p = p < 0 ? 0 : (p >= max_ctx ? max_ctx - 1 : p);
  const int n = (int)p + 1;
  if (row0 >= n) return;  // nothing to look at: the combining kernel skips this split as well
  if constexpr (ROPE) {
    const half8 cv = *reinterpret_cast<const half8*>(cos_t + (size_t)p * d + sub * 8);
    const half8 sv = *reinterpret_cast<const half8*>(sin_t + (size_t)p * d + sub * 8);
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const float ko = (float)k_cur[e];
      const float kp = __shfl_xor(ko, 8, 64);
      k_cur[e] = rotary(ko, sub < 8 ? -kp : kp, cv[e], sv[e]);
#pragma unroll
      for (int r = 0; r < REP; r++) {
        const float qo = (float)qv[r][e];
        const float qp = __shfl_xor(qo, 8, 64);
        qv[r][e] = rotary(qo, sub < 8 ? -qp : qp, cv[e], sv[e]);
      }
    }
    // the workgroup whose rows include the new one writes it to the caches
    if ((int)p >= row0 && (int)p < row0 + kSplitRows && grp == 0) {
      *reinterpret_cast<half8*>(k_cache + ((size_t)kvh * max_ctx + p) * d + sub * 8) = k_cur;
      *reinterpret_cast<half8*>(v_cache + ((size_t)kvh * max_ctx + p) * d + sub * 8) = v_cur;
    }
  }
#pragma unroll
  for (int u = 0; u < 4; u++) {
    const int t = row0 + grp + 16 * u;
    const half8 kk = ROPE && t == (int)p ? k_cur : kr[u];
#pragma unroll
    for (int r = 0; r < REP; r++) {
      float dot = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e++) dot += (float)qv[r][e] * scale * (float)kk[e];
#pragma unroll
      for (int o = 8; o > 0; o >>= 1) dot += __shfl_xor(dot, o, 64);
      if (sub == 0) sc[r][grp + 16 * u] = t < n ? dot : -INFINITY;
    }
  }
  __syncthreads();
  // maximum and sum of exponentials per query head: wave w takes heads w, w + 4; lane = row
  for (int r = wave; r < REP; r += 4) {
    const float v = sc[r][lane];
    const float mx = wave_max(v);
    const float e = mx == -INFINITY ? 0.f : __expf(v - mx);
    sc[r][lane] = e;
    const float sum = wave_sum(e);
    if (lane == 0) { mx_s[r] = mx; sum_s[r] = sum; }
  }
  __syncthreads();
  float acc[REP][8];
#pragma unroll
  for (int r = 0; r < REP; r++)
#pragma unroll
    for (int e = 0; e < 8; e++) acc[r][e] = 0.f;
#pragma unroll
  for (int u = 0; u < 4; u++) {
    const int t = row0 + grp + 16 * u;
    if (t < n) {  // (an unused row may hold anything, also NaN)
      const half8 vv = ROPE && t == (int)p ? v_cur : vr[u];
#pragma unroll
      for (int r = 0; r < REP; r++) {
        const float pr = sc[r][grp + 16 * u];
#pragma unroll
        for (int e = 0; e < 8; e++) acc[r][e] += pr * (float)vv[e];
      }
    }
  }
  // the four row groups of a wave by shuffles, the four waves through LDS
#pragma unroll
  for (int r = 0; r < REP; r++)
#pragma unroll
    for (int e = 0; e < 8; e++) {
      acc[r][e] += __shfl_xor(acc[r][e], 16, 64);
      acc[r][e] += __shfl_xor(acc[r][e], 32, 64);
    }
  if (lane < 16) {
#pragma unroll
    for (int r = 0; r < REP; r++)
#pragma unroll
      for (int e = 0; e < 8; e++) part[wave][r][sub * 8 + e] = acc[r][e];
  }
  __syncthreads();
  const int head0 = kvh * REP;
  for (int idx = tid; idx < REP * d; idx += 256) {
    const int r = idx >> 7, dim = idx & 127;
    float* dst = ws + ((size_t)(m * heads + head0 + r) * splits + split) * kSplitStride;
    dst[dim] = part[0][r][dim] + part[1][r][dim] + part[2][r][dim] + part[3][r][dim];
    if (dim == 0) { dst[128] = mx_s[r]; dst[129] = sum_s[r]; }
  }
}

// out[m, head, :] = sum over the splits with rows (those below pos[m] + 1) of the partial values,
// each weighted by exp(its maximum - the overall maximum), over the sum of the partial sums
// weighted alike.  Grid (heads, M), 128 threads (one per element of the head).
__global__ void __launch_bounds__(128)
attention_combine_kernel(const float* __restrict__ ws, const int64_t* __restrict__ pos, _Float16* __restrict__ out,
                         int heads, int64_t max_ctx, int splits) {
  constexpr int d = 128;
  const int head = blockIdx.x, m = blockIdx.y, dim = threadIdx.x;
  int64_t p = pos[m];
  p = p < 0 ? 0 : (p >= max_ctx ? max_ctx - 1 : p);
  const int used = ((int)p + kSplitRows) / kSplitRows;  // splits that hold rows 0 .. p
  const float* src = ws + (size_t)(m * heads + head) * splits * kSplitStride;
  // eight splits at a time, all their loads in flight together (a split beyond the used ones
  // re-reads the last used one with weight zero); running maximum, sum and value are rescaled
  // whenever a chunk raises the maximum
  float mx = -INFINITY, sum = 0.f, o = 0.f;
  for (int sp0 = 0; sp0 < used; sp0 += 8) {
    float ms[8], ls[8], vs[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const float* part = src + (size_t)(sp0 + i < used ? sp0 + i : used - 1) * kSplitStride;
      ms[i] = part[128];
      ls[i] = part[129];
      vs[i] = part[dim];
    }
    float cm = mx;
#pragma unroll
    for (int i = 0; i < 8; i++) cm = fmaxf(cm, ms[i]);
    const float keep = mx == -INFINITY ? 0.f : __expf(mx - cm);
    sum *= keep;
    o *= keep;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const float w = sp0 + i < used ? __expf(ms[i] - cm) : 0.f;
      sum += w * ls[i];
      o += w * vs[i];
    }
    mx = cm;
  }
  out[((size_t)m * heads + head) * d + dim] = (_Float16)(o / sum);
}

template <bool ROPE>
int launch_attention_split(const void* qkv, void* k_cache, void* v_cache, const int64_t* pos, void* out,
                           const void* cos_table, const void* sin_table, void* ws, int64_t M, int heads,
                           int kv_heads, int64_t max_ctx, void* stream) {
  const int splits = (int)((max_ctx + kSplitRows - 1) / kSplitRows);
  const dim3 grid((unsigned)kv_heads, (unsigned)splits, (unsigned)M), block(256);
  const float scale = 1.0f / sqrtf(128.0f);
#define MATGPTQ_GLUE_SPLIT(REP)                                                                              \
  hipLaunchKernelGGL((attention_split_kernel<ROPE, REP>), grid, block, 0, (hipStream_t)stream,                \
                     (const _Float16*)qkv, (_Float16*)k_cache, (_Float16*)v_cache, pos, (_Float16*)out,       \
                     (const _Float16*)cos_table, (const _Float16*)sin_table, (float*)ws, heads, kv_heads,   \
                     max_ctx, splits, scale)
  switch (heads / kv_heads) {
    case 1: MATGPTQ_GLUE_SPLIT(1); break;
    case 2: MATGPTQ_GLUE_SPLIT(2); break;
    case 4: MATGPTQ_GLUE_SPLIT(4); break;
    case 8: MATGPTQ_GLUE_SPLIT(8); break;
    default: return MATGPTQ_GLUE_ESHAPE;
  }
#undef MATGPTQ_GLUE_SPLIT
  if (int e = launch_status()) return e;
  hipLaunchKernelGGL(attention_combine_kernel, dim3((unsigned)heads, (unsigned)M), dim3(128), 0,
                     (hipStream_t)stream, (const float*)ws, pos, (_Float16*)out, heads, max_ctx, splits);
  return launch_status();
}

// out[m, j] = silu(gu[m, j]) * gu[m, F + j]; both factors rounded to fp16 like the two
// element-wise operators it replaces.
__global__ void __launch_bounds__(kThreads)
silu_mul_kernel(const _Float16* __restrict__ gu, _Float16* __restrict__ out, int64_t M, int64_t F) {
  const int64_t per_row = F / 8;
  const int64_t c = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (c >= M * per_row) return;
  const int64_t m = c / per_row, j = c - m * per_row;
  const half8 g = *reinterpret_cast<const half8*>(gu + m * 2 * F + j * 8);
  const half8 u = *reinterpret_cast<const half8*>(gu + m * 2 * F + F + j * 8);
  half8 o;
#pragma unroll
  for (int e = 0; e < 8; e++) {
    const float x = (float)g[e];
    const _Float16 s = (_Float16)(x / (1.0f + __expf(-x)));
    o[e] = s * u[e];
  }
  *reinterpret_cast<half8*>(out + m * F + j * 8) = o;
}

// Index of the largest value of each row of x [M, n] (fp32): the first one among equals, a NaN counts
// as the largest, like torch.argmax.  One workgroup per row: the library's reduction spends 38 us in
// one workgroup of 512 threads on a vocabulary of 128256; sixteen waves with eight 16-byte loads in
// flight per thread read the same 0.5 MB in a few microseconds.
constexpr int kArgmaxThreads = 1024;
__device__ __forceinline__ bool argmax_better(float v, int i, float bv, int bi) {
  const bool vn = v != v, bn = bv != bv;
  if (vn != bn) return vn;
  if (vn) return i < bi;
  return v > bv || (v == bv && i < bi);
}
__global__ void __launch_bounds__(kArgmaxThreads)
argmax_kernel(const float* __restrict__ x, int64_t* __restrict__ out, int64_t n) {
  __shared__ float sv[kArgmaxThreads / 64];
  __shared__ int si[kArgmaxThreads / 64];
  const float* row = x + (size_t)blockIdx.x * (size_t)n;
  float best = -INFINITY;
  int bi = 0x7fffffff;
  // whole float4 chunks when the row starts on 16 bytes, element by element otherwise and at the end
  const bool aligned = (reinterpret_cast<uintptr_t>(row) & 15) == 0;
  const int chunks = aligned ? (int)(n / 4) : 0;
  constexpr int kDepth = 8;
  for (int c0 = threadIdx.x; c0 < chunks; c0 += kArgmaxThreads * kDepth) {
    float4 v[kDepth];
#pragma unroll
    for (int u = 0; u < kDepth; u++) {  // (unconditional: a chunk past the end re-reads the last one, which changes nothing)
      const int c = c0 + u * kArgmaxThreads;
      v[u] = reinterpret_cast<const float4*>(row)[c < chunks ? c : chunks - 1];
    }
#pragma unroll
    for (int u = 0; u < kDepth; u++) {
      const int c = c0 + u * kArgmaxThreads < chunks ? c0 + u * kArgmaxThreads : chunks - 1;
      const float e[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
      // a thread meets its indices in rising order: "greater" alone keeps the first of equals
#pragma unroll
      for (int k = 0; k < 4; k++)
        if (e[k] > best || (e[k] != e[k] && best == best)) { best = e[k]; bi = 4 * c + k; }
    }
  }
  for (int i = chunks * 4 + threadIdx.x; i < n; i += kArgmaxThreads) {
    const float e = row[i];
    if (e > best || (e != e && best == best)) { best = e; bi = i; }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(bi, o, 64);
    if (argmax_better(ov, oi, best, bi)) { best = ov; bi = oi; }
  }
  if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = best; si[threadIdx.x >> 6] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kArgmaxThreads / 64; w++)
      if (argmax_better(sv[w], si[w], best, bi)) { best = sv[w]; bi = si[w]; }
    out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;  // (a row of -inf only: nothing was greater than the start value)
  }
}

}  // namespace

extern "C" {

int matgptq_glue_add_rmsnorm(void* h, const void* delta, const void* weight, void* x, int64_t M, int64_t H,
                             float eps, void* stream) {
  if (!h || !weight || !x) return MATGPTQ_GLUE_ENULL;
  if (M <= 0 || H <= 0 || H % 8 != 0) return MATGPTQ_GLUE_ESHAPE;
  if (H > 8 * kThreads * kMaxChunks || M > 65535) return MATGPTQ_GLUE_ESIZE;
  hipLaunchKernelGGL(add_rmsnorm_kernel, dim3((unsigned)M), dim3(kThreads), 0, (hipStream_t)stream,
                     (_Float16*)h, (const _Float16*)delta, (const _Float16*)weight, (_Float16*)x, (int)H, eps);
  return launch_status();
}

int matgptq_glue_rope_cache(void* qkv, const void* cos_table, const void* sin_table, const int64_t* pos,
                            void* k_cache, void* v_cache, int64_t M, int heads, int kv_heads, int head_dim,
                            int64_t max_ctx, void* stream) {
  if (!qkv || !cos_table || !sin_table || !pos || !k_cache || !v_cache) return MATGPTQ_GLUE_ENULL;
  if (M <= 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || head_dim <= 0 || head_dim % 2 != 0 ||
      max_ctx <= 0)
    return MATGPTQ_GLUE_ESHAPE;
  if (M > 65535) return MATGPTQ_GLUE_ESIZE;
  hipLaunchKernelGGL(rope_cache_kernel, dim3((unsigned)(heads + 2 * kv_heads), (unsigned)M), dim3(64), 0,
                     (hipStream_t)stream, (_Float16*)qkv, (const _Float16*)cos_table, (const _Float16*)sin_table,
                     pos, (_Float16*)k_cache, (_Float16*)v_cache, heads, kv_heads, head_dim, max_ctx);
  return launch_status();
}

int matgptq_glue_attention(const void* qkv, const void* k_cache, const void* v_cache, const int64_t* pos,
                           void* out, int64_t M, int heads, int kv_heads, int head_dim, int64_t max_ctx,
                           void* stream) {
  if (!qkv || !k_cache || !v_cache || !pos || !out) return MATGPTQ_GLUE_ENULL;
  if (M <= 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || head_dim != 128 || max_ctx <= 0)
    return MATGPTQ_GLUE_ESHAPE;
  if (M > 65535 || max_ctx > MATGPTQ_GLUE_MAX_CONTEXT) return MATGPTQ_GLUE_ESIZE;
  const size_t lds = ((size_t)max_ctx + kAttnWaves * 128 + kAttnWaves) * sizeof(float);
  hipLaunchKernelGGL(attention_kernel<false>, dim3((unsigned)heads, (unsigned)M), dim3(kAttnThreads), lds,
                     (hipStream_t)stream, (const _Float16*)qkv, (_Float16*)k_cache, (_Float16*)v_cache, pos,
                     (_Float16*)out, (const _Float16*)nullptr, (const _Float16*)nullptr, heads, kv_heads,
                     max_ctx, 1.0f / sqrtf((float)head_dim));
  return launch_status();
}

int matgptq_glue_rope_attention(const void* qkv, const void* cos_table, const void* sin_table,
                                const int64_t* pos, void* k_cache, void* v_cache, void* out, int heads,
                                int kv_heads, int head_dim, int64_t max_ctx, void* stream) {
  if (!qkv || !cos_table || !sin_table || !pos || !k_cache || !v_cache || !out) return MATGPTQ_GLUE_ENULL;
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || head_dim != 128 || max_ctx <= 0)
    return MATGPTQ_GLUE_ESHAPE;
  if (max_ctx > MATGPTQ_GLUE_MAX_CONTEXT) return MATGPTQ_GLUE_ESIZE;
  const size_t lds = ((size_t)max_ctx + kAttnWaves * 128 + kAttnWaves) * sizeof(float);
  hipLaunchKernelGGL(attention_kernel<true>, dim3((unsigned)heads, 1u), dim3(kAttnThreads), lds,
                     (hipStream_t)stream, (const _Float16*)qkv, (_Float16*)k_cache, (_Float16*)v_cache, pos,
                     (_Float16*)out, (const _Float16*)cos_table, (const _Float16*)sin_table, heads, kv_heads,
                     max_ctx, 1.0f / sqrtf((float)head_dim));
  return launch_status();
}

size_t matgptq_glue_attention_workspace_floats(int64_t M, int heads, int64_t max_ctx) {
  if (M <= 0 || heads <= 0 || max_ctx <= 0) return 0;
  return (size_t)M * heads * ((max_ctx + kSplitRows - 1) / kSplitRows) * kSplitStride;
}

int matgptq_glue_attention_split(const void* qkv, const void* cos_table, const void* sin_table,
                                 const int64_t* pos, void* k_cache, void* v_cache, void* out, void* workspace,
                                 int64_t M, int heads, int kv_heads, int head_dim, int64_t max_ctx,
                                 int fuse_rotary, void* stream) {
  if (!qkv || !pos || !k_cache || !v_cache || !out || !workspace) return MATGPTQ_GLUE_ENULL;
  if (fuse_rotary && (!cos_table || !sin_table)) return MATGPTQ_GLUE_ENULL;
  if (M <= 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || head_dim != 128 || max_ctx <= 0 ||
      (fuse_rotary && M != 1))
    return MATGPTQ_GLUE_ESHAPE;
  if (M > 65535 || max_ctx > MATGPTQ_GLUE_MAX_CONTEXT) return MATGPTQ_GLUE_ESIZE;
  return fuse_rotary ? launch_attention_split<true>(qkv, k_cache, v_cache, pos, out, cos_table, sin_table,
                                                    workspace, M, heads, kv_heads, max_ctx, stream)
                     : launch_attention_split<false>(qkv, k_cache, v_cache, pos, out, cos_table, sin_table,
                                                     workspace, M, heads, kv_heads, max_ctx, stream);
}

int matgptq_glue_argmax(const void* x, void* out, int64_t M, int64_t n, void* stream) {
  if (!x || !out) return MATGPTQ_GLUE_ENULL;
  if (M <= 0 || n <= 0) return MATGPTQ_GLUE_ESHAPE;
  if (M > 65535 || n > 0x7fffffff) return MATGPTQ_GLUE_ESIZE;
  hipLaunchKernelGGL(argmax_kernel, dim3((unsigned)M), dim3(kArgmaxThreads), 0, (hipStream_t)stream,
                     (const float*)x, (int64_t*)out, n);
  return launch_status();
}

int matgptq_glue_silu_mul(const void* gate_up, void* out, int64_t M, int64_t F, void* stream) {
  if (!gate_up || !out) return MATGPTQ_GLUE_ENULL;
  if (M <= 0 || F <= 0 || F % 8 != 0) return MATGPTQ_GLUE_ESHAPE;
  const int64_t blocks = (M * (F / 8) + kThreads - 1) / kThreads;
  if (blocks > 0x7fffffff) return MATGPTQ_GLUE_ESIZE;
  hipLaunchKernelGGL(silu_mul_kernel, dim3((unsigned)blocks), dim3(kThreads), 0, (hipStream_t)stream,
                     (const _Float16*)gate_up, (_Float16*)out, M, F);
  return launch_status();
}

const char* matgptq_glue_strerror(int code) {
  switch (code) {
    case 0: return "ok";
    case MATGPTQ_GLUE_ESHAPE: return "a size is not positive or not divisible as the operator requires";
    case MATGPTQ_GLUE_ENULL: return "a required pointer is NULL";
    case MATGPTQ_GLUE_ELAUNCH: return "the HIP runtime reported an error at launch";
    case MATGPTQ_GLUE_ESIZE: return "a size exceeds what the operator supports";
    default: return "unknown error";
  }
}

}  // extern "C"
