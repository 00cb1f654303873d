/* Decode-time operators between the bit-sliced linears of a decoder block
 * (libmatgptq_glue.so, built from matgptq_amd/csrc/glue_gfx950.hip).
 *
 * These have no counterpart in the reference's extension: the reference leaves norms,
 * rotary embedding, attention and the activation to transformers / vLLM
 * (inference_lib/inference_demo_transformers.py:134-176,
 *  inference_lib/bench_transformers_e2e.py:61-76).  They exist for the end-to-end
 * tokens/s measurement of a Mix'n'Match decoder, where those operators as separate
 * library kernels cost more than the linears, and they are kept out of the GEMM's
 * drop-in library (include/matgptq_abi.h) on purpose.
 *
 * Plain C ABI: device pointers, sizes, a HIP stream; fp16 storage, fp32 arithmetic.
 * Every call is asynchronous on `stream`, allocates nothing and reads nothing on the
 * host (graph-capturable).  Returns 0 or a negative MATGPTQ_GLUE_E* code. */
#ifndef MATGPTQ_GLUE_H
#define MATGPTQ_GLUE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MATGPTQ_GLUE_ESHAPE (-3)  /* a size is not positive or not divisible as required */
#define MATGPTQ_GLUE_ENULL (-4)   /* a required pointer is NULL */
#define MATGPTQ_GLUE_ELAUNCH (-6) /* the HIP runtime reported an error at launch */
#define MATGPTQ_GLUE_ESIZE (-8)   /* a size exceeds what the operator supports */

/* longest cache the attention operator takes (its scores wait in LDS) */
#define MATGPTQ_GLUE_MAX_CONTEXT 8192

const char *matgptq_glue_strerror(int code);

/* h[M,H] += delta[M,H] (skipped when delta is NULL), then
 * x[M,H] = h * rsqrt(mean(h^2) + eps) * weight[H].  H % 8 == 0, H <= 8192. */
int matgptq_glue_add_rmsnorm(void *h, const void *delta, const void *weight, void *x,
                             int64_t M, int64_t H, float eps, void *stream);

/* qkv[M, (heads + 2 kv_heads) * head_dim]: rotary embedding (half-split pairs, angles of
 * row pos[m] of cos_table / sin_table [max_ctx, head_dim]) of the query heads in place and
 * of the key heads into k_cache[kv_heads, max_ctx, head_dim] at row pos[m]; the value heads
 * are copied to the same row of v_cache.  pos: int64 [M], clamped to the cache. */
int matgptq_glue_rope_cache(void *qkv, const void *cos_table, const void *sin_table,
                            const int64_t *pos, void *k_cache, void *v_cache, int64_t M,
                            int heads, int kv_heads, int head_dim, int64_t max_ctx, void *stream);

/* out[M, heads * head_dim] = softmax(q k^T / sqrt(head_dim)) v for the (rotated) query heads
 * in qkv, each row m over the cache rows 0 .. pos[m]; grouped-query heads share a cache
 * head.  head_dim == 128, max_ctx <= MATGPTQ_GLUE_MAX_CONTEXT.  Meant for a few rows. */
int matgptq_glue_attention(const void *qkv, const void *k_cache, const void *v_cache,
                           const int64_t *pos, void *out, int64_t M, int heads, int kv_heads,
                           int head_dim, int64_t max_ctx, void *stream);

/* matgptq_glue_rope_cache followed by matgptq_glue_attention for a single row (M = 1) in one
 * launch, with the same results: qkv is read only (the rotated query stays in registers),
 * k_cache and v_cache receive row pos[0], out[1, heads * head_dim] the attention output. */
int matgptq_glue_rope_attention(const void *qkv, const void *cos_table, const void *sin_table,
                                const int64_t *pos, void *k_cache, void *v_cache, void *out,
                                int heads, int kv_heads, int head_dim, int64_t max_ctx,
                                void *stream);

/* The same attention with the context split over workgroups (one per key/value head and 64
 * cache rows, serving all query heads of that key/value head) and a second small launch that
 * combines their partial results: for short batches, where a workgroup per query head leaves
 * most of the GPU idle.  Query heads per key/value head: 1, 2, 4 or 8.  fuse_rotary != 0 (M = 1
 * only) also does what matgptq_glue_rope_cache does, like matgptq_glue_rope_attention;
 * otherwise qkv holds rotated queries and the caches are read only (cos_table / sin_table may
 * be NULL).  workspace: matgptq_glue_attention_workspace_floats() floats, contents irrelevant
 * before and after; calls that share a workspace must not overlap.  Results agree with
 * matgptq_glue_attention to the fp32 rounding of the softmax sums. */
size_t matgptq_glue_attention_workspace_floats(int64_t M, int heads, int64_t max_ctx);
int matgptq_glue_attention_split(const void *qkv, const void *cos_table, const void *sin_table,
                                 const int64_t *pos, void *k_cache, void *v_cache, void *out,
                                 void *workspace, int64_t M, int heads, int kv_heads,
                                 int head_dim, int64_t max_ctx, int fuse_rotary, void *stream);

/* out[m] (int64) = index of the largest of x[m, 0:n] (fp32, rows contiguous): the first among equals, a NaN
 * counts as the largest (torch.argmax).  One launch, no workspace.  M <= 65535, n < 2^31. */
int matgptq_glue_argmax(const void *x, void *out, int64_t M, int64_t n, void *stream);

/* out[M,F] = silu(gate_up[M, 0:F]) * gate_up[M, F:2F].  F % 8 == 0. */
int matgptq_glue_silu_mul(const void *gate_up, void *out, int64_t M, int64_t F, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MATGPTQ_GLUE_H */
