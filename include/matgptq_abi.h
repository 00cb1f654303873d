/*
 * C ABI of the MI355X (gfx950) implementation of MatGPTQ's bit-sliced GEMM.
 *
 * Plain pointers and sizes only; no torch types.  Every function returns 0 on
 * success or a negative MATGPTQ_E* code (never exits the process, never
 * synchronises the device unless the SYNC convention below asks for it).
 * `stream` is a hipStream_t passed as void* (NULL = the default stream).
 * Pointers named *_dev are device memory, *_host are host memory.
 *
 * Naming of sizes follows torch.nn.Linear: W is [N, K] (out x in), X is [M, K],
 * Y = X * W^T is [M, N].  The reference calls them m (=N), n (=K), k (=M).
 *
 * Preconditions shared by all entry points: bitwidth in {2,3,4,6,8},
 * group_size in {-1,32,128}, N % 16 == 0, K % 128 == 0 or (group sizes 32 and -1) K % 128 == 64
 * with K >= 192 (the reference: K % 64 == 0, inference_lib/matgptq_cuda/csrc/utils.cpp:174-184);
 * the master-resident entry points take K % 128 == 0 only.
 */
#ifndef MATGPTQ_ABI_H
#define MATGPTQ_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MATGPTQ_ABI_VERSION 2

/* error codes */
#define MATGPTQ_OK 0
#define MATGPTQ_EBITS (-1)     /* bitwidth not in {2,3,4,6,8} */
#define MATGPTQ_EGROUP (-2)    /* group_size not in {-1,32,128} or does not divide K */
#define MATGPTQ_ESHAPE (-3)    /* N % 16 != 0, K not of the forms above, or a size <= 0 */
#define MATGPTQ_ENULL (-4)     /* a required pointer is NULL */
#define MATGPTQ_EDTYPE (-5)    /* operation not available for the requested data type */
#define MATGPTQ_ELAUNCH (-6)   /* the HIP runtime reported an error at launch */
#define MATGPTQ_EVARIANT (-7)  /* a forced kernel variant does not apply to this problem */
#define MATGPTQ_ESIZE (-8)     /* a size exceeds what the entry point supports */
#define MATGPTQ_EWORKSPACE (-9) /* workspace missing or too small */
#define MATGPTQ_ESTATIC (-10)   /* needs more than the library's built-in workspace */
#define MATGPTQ_EALIAS (-11)    /* an output buffer overlaps an input that other workgroups still read */

/* feature_flag bits: the reference's `Features` word
 * (inference_lib/matgptq_cuda/csrc/include/common.cuh:78-86,
 *  inference_lib/matgptq_cuda/matgptq_linear.py:6-9). */
#define MATGPTQ_FLAG_ASYNC 1u /* bit 0: 1 = do not synchronise after the launch */
#define MATGPTQ_FLAG_BF16 2u  /* bit 1: activations / scales / output are bf16 */
/* Bits 8..17: benchmark-only override of the kernel choice (0 = automatic).  Bits 8..15:
 * 1..42 decode kernel (work split), 64..79, 89 and 90 prefill tile, 80..88 and 91 mid-batch kernel (row blocks
 * and batch rows per workgroup); bits 16..17: decode flavour (1 burst, 2 stream), which also
 * keeps small batches on the decode kernel.  A value that does not apply returns
 * MATGPTQ_EVARIANT. */
#define MATGPTQ_FLAG_VARIANT_SHIFT 8
#define MATGPTQ_FLAG_VARIANT_MASK 0xFF00u
#define MATGPTQ_FLAG_FLAVOUR_SHIFT 16
#define MATGPTQ_FLAG_FLAVOUR_MASK 0x30000u
/* gemv kernel (batch 1..4; 5..8 with one scale per tile or row, entries 1 and 2; variant 100 + entry): bits 18..22 waves per workgroup
 * (0 = automatic), bits 23..28 dynamic LDS to request, in units of 4 KiB (0 = what it needs) */
#define MATGPTQ_FLAG_GEMV_WAVES_SHIFT 18
#define MATGPTQ_FLAG_GEMV_LDS_SHIFT 23

int matgptq_abi_version(void);
const char *matgptq_strerror(int code);

/* Number of uint32 words of a packed weight: bitwidth*N*K/32, the size the
 * reference's op checks (inference_lib/matgptq_cuda/csrc/bindings.cpp:68,160).
 * Returns 0 for invalid arguments. */
size_t matgptq_packed_words(int bitwidth, int64_t N, int64_t K);

/* ---- the GEMM ------------------------------------------------------------
 * Replaces MATGPTQ_CUDA::matmul_matgptq_host
 * (inference_lib/matgptq_cuda/csrc/include/gemm.h:22-32,
 *  inference_lib/matgptq_cuda/csrc/matgptq_gemm.cu:1026-1065).
 *
 *   Y[M,N] = fp16( sum_k X[m,k] * scale[n,k/g] * ((c[n,k] << (8-b)) - zero[n,k/g]) )
 *
 * packed_dev   output of matgptq_pack_* (b-bit codes c, already sliced)
 * scales_dev   output of matgptq_reorder_scales_* applied to scale[N, K/g] (fp16)
 * zeros_dev    output of matgptq_reorder_scales_* applied to zero[N, K/g] (fp16),
 *              or NULL: every zero is 128, which is the reference kernel's
 *              symmetric form  (c - 2^(b-1)) * scale * 2^(8-b)
 * x_dev        [M, K] fp16 row-major;  y_dev  [M, N] fp16 row-major
 * Any M >= 1 is accepted.  Graph-capturable: no allocation, no host read.
 * With flag bit 0 clear the call ends with hipStreamSynchronize(stream). */
int matgptq_gemm(int bitwidth, int group_size, int64_t N, int64_t K, int64_t M,
                 const void *packed_dev, const void *scales_dev, const void *zeros_dev,
                 const void *x_dev, void *y_dev, void *stream, uint32_t flags);

/* ---- packing on the host ---------------------------------------------------
 * Replaces swizzle_weights / split_up_n_bits / swizzle_matgptq
 * (inference_lib/matgptq_cuda/csrc/utils.cpp:22-217) as driven by
 * pack_matgptq_qweights (inference_lib/matgptq_cuda/csrc/bindings.cpp:43-84).
 * codes_host: uint8 [N, K].  If slice_from_master != 0 the codes are 8-bit
 * master codes and are first sliced to `bitwidth` with the reference's rounded
 * slice (src/quant_utils_matgpqt.py:9-17); otherwise they must already be
 * < 2^bitwidth (higher bits are ignored).  out_host: matgptq_packed_words() words. */
int matgptq_pack_host(const uint8_t *codes_host, int64_t N, int64_t K, int bitwidth,
                      int slice_from_master, uint32_t *out_host);

/* Inverse of matgptq_pack_host (tests, bit-exactness checks). */
int matgptq_unpack_host(const uint32_t *packed_host, int64_t N, int64_t K, int bitwidth,
                        uint8_t *codes_host);

/* Replaces reorder_matgptq_scales (inference_lib/matgptq_cuda/csrc/bindings.cpp:86-142).
 * in: 16-bit elements [N, G] (G = K/g, 1 for g = -1); out: same count, ordered
 * [N/16][G][16] so that the 16 rows of a tile are contiguous per group.
 * Works on any 16-bit type (fp16 scales, fp16 zeros, bf16). */
int matgptq_reorder_scales_host(const uint16_t *in_host, int64_t N, int64_t K, int group_size,
                                uint16_t *out_host);

/* ---- packing on the device ---------------------------------------------------
 * Same results as the host functions, for tensors that already live in HBM
 * (the reference copies to the host and back, bindings.cpp:70-83,99-141).
 * Asynchronous on `stream`. */
int matgptq_pack_device(const uint8_t *codes_dev, int64_t N, int64_t K, int bitwidth,
                        int slice_from_master, uint32_t *out_dev, void *stream);
int matgptq_unpack_device(const uint32_t *packed_dev, int64_t N, int64_t K, int bitwidth,
                          uint8_t *codes_dev, void *stream);
int matgptq_reorder_scales_device(const uint16_t *in_dev, int64_t N, int64_t K, int group_size,
                                  uint16_t *out_dev, void *stream);

/* Rounded MSB slice of master codes on the device, element-wise
 * (src/quant_utils_matgpqt.py:9-17 with master_bitwidth = 8). */
int matgptq_slice_device(const uint8_t *master_dev, int64_t count, int bitwidth,
                         uint8_t *sliced_dev, void *stream);

/* Dequantised weight W[N,K] (fp16) from a packed tensor, rounded once per
 * element exactly like the reference's dequantize (src/quant_utils_matgpqt.py:19-22).
 * Used by tests and by callers that want a dense copy. */
int matgptq_dequantize_device(int bitwidth, int group_size, int64_t N, int64_t K,
                              const void *packed_dev, const void *scales_dev,
                              const void *zeros_dev, void *w_dev, void *stream);

/* ---- decode with the operator in front of the linear fused into it ---------------------
 * No counterpart in the reference, whose callers run these as separate element-wise kernels between
 * the linears (the transformers model of inference_lib/inference_demo_transformers.py:132-175; each
 * costs a launch and a round trip through memory, more than a decode GEMV of the smaller layers).
 * matgptq_gemm with the activations formed while the kernel stages them; fp16 storage, group size
 * 128, 1 <= M <= 4 (the batch-1..4 kernel), pre-sliced codes:
 *   MATGPTQ_PRE_SILU_MUL     a_dev is [M, 2K] (gate | up, as the fused gate_up linear leaves them):
 *                            x = fp16(silu(gate)) * up, the roundings of two element-wise operators;
 *                            b_dev, w_dev, out_dev unused.
 *   MATGPTQ_PRE_ADD_RMSNORM  a_dev is the residual stream h [M, K], b_dev what is added to it [M, K]
 *                            (or NULL), w_dev the norm's weight [K]:  v = h + b (one fp16 rounding),
 *                            x = fp16(v * rsqrt(mean(v^2) + eps) * w);  v is also written to out_dev
 *                            [M, K] when that is not NULL.  out_dev must not overlap a_dev or b_dev
 *                            (MATGPTQ_EALIAS): other workgroups still read them.  K <= 8192.
 * Shapes outside these limits return MATGPTQ_EVARIANT: run the operator and matgptq_gemm separately. */
#define MATGPTQ_PRE_SILU_MUL 1
#define MATGPTQ_PRE_ADD_RMSNORM 2
int matgptq_gemm_prologue(int bitwidth, int group_size, int64_t N, int64_t K, int64_t M,
                          const void *packed_dev, const void *scales_dev, const void *zeros_dev,
                          int kind, const void *a_dev, const void *b_dev, const void *w_dev, void *out_dev,
                          float eps, void *y_dev, void *stream, uint32_t flags);

/* Measurement aid (no counterpart in the reference): streams `bytes` of device memory once through
 * the load pattern of the batch-1 kernel (a wave requests four KiB-sized pieces at once, eight
 * waves per workgroup) and does nothing with them.  bench.py times it on buffers of the size of a
 * layer to state what a kernel that only read the weights would take on the same GPU. */
int matgptq_probe_read(const void *buf_dev, size_t bytes, void *stream);

/* ---- master-resident codes ------------------------------------------------------
 * The reference slices the 8-bit master codes once on the host, packs the slice and deletes
 * the master codes (inference_lib/vllm_matgptq.py:154-178,
 * inference_lib/inference_demo_transformers.py:30-40): another bitwidth needs the checkpoint
 * again.  Here the master codes can stay resident as bit planes, most significant first
 * (N*K/4 words), and the GEMM takes the bitwidth as an argument: it reads the top `bitwidth`
 * bits of every code plus the bit below them and forms the reference's rounded, saturating
 * slice (src/quant_utils_matgpqt.py:9-17) in registers.  (bitwidth + 1)/8 bytes per weight
 * are moved for 2, 3 and 4 bits, one byte for 6 and 8. */
size_t matgptq_master_words(int64_t N, int64_t K); /* N*K/4, 0 for invalid arguments */
int matgptq_pack_master_host(const uint8_t *codes_host, int64_t N, int64_t K, uint32_t *planes_host);
int matgptq_pack_master_device(const uint8_t *codes_dev, int64_t N, int64_t K, uint32_t *planes_dev,
                               void *stream);
/* The codes the GEMM sees at `bitwidth`: uint8 [N, K], sliced with the same instruction
 * sequence the kernels run (bit-exactness checks against matryoshka_slice). */
int matgptq_unpack_master_host(const uint32_t *planes_host, int64_t N, int64_t K, int bitwidth,
                               uint8_t *codes_host);
int matgptq_unpack_master_device(const uint32_t *planes_dev, int64_t N, int64_t K, int bitwidth,
                                 uint8_t *codes_dev, void *stream);
/* matgptq_gemm on master-resident planes.  Batch sizes 1..4 (the HBM-bound regime, where the
 * bytes moved decide) and the mid-batch kernel - every shape up to 128 batch rows, and the larger
 * batches that kernel is planned for anyway - read the planes in the GEMM kernel itself.  Every other
 * shape slices the planes into the pre-sliced layout first, in `workspace_dev`
 * (matgptq_gemm_master_workspace_bytes() bytes, 0 when none is needed), and runs the kernel of that
 * regime on it: two launches, no allocation.  Too small a workspace returns MATGPTQ_EWORKSPACE. */
size_t matgptq_gemm_master_workspace_bytes(int bitwidth, int group_size, int64_t N, int64_t K, int64_t M,
                                           uint32_t flags);
int matgptq_gemm_master(int bitwidth, int group_size, int64_t N, int64_t K, int64_t M,
                        const void *planes_dev, const void *scales_dev, const void *zeros_dev,
                        const void *x_dev, void *y_dev, void *workspace_dev, size_t workspace_bytes,
                        void *stream, uint32_t flags);

/* matgptq_gemm_master without a workspace argument and without any allocation.  It has no
 * counterpart in the reference; it is for callers that cannot allocate or carry a workspace along:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  Where
 * matgptq_gemm_master would use its workspace, this entry point uses a buffer of
 * MATGPTQ_STATIC_WORKSPACE_BYTES that is part of the library's device code (every GPU the library
 * runs on holds one copy until the process ends).  A shape whose sliced tensor
 * (bitwidth*N*K/8 bytes) does not fit returns MATGPTQ_ESTATIC.  All calls on one GPU share that
 * buffer: calls that overlap in time on one GPU (different streams) race, calls on one stream do
 * not.  The first call on a device looks the buffer's address up (hipGetSymbolAddress), so make
 * that call outside graph capture. */
#define MATGPTQ_STATIC_WORKSPACE_BYTES (64u * 1024u * 1024u)
int matgptq_gemm_master_static(int bitwidth, int group_size, int64_t N, int64_t K, int64_t M,
                               const void *planes_dev, const void *scales_dev, const void *zeros_dev,
                               const void *x_dev, void *y_dev, void *stream, uint32_t flags);

/* Human-readable name of the kernel variant matgptq_gemm would launch. */
int matgptq_describe_plan(int bitwidth, int group_size, int64_t N, int64_t K, int64_t M,
                          int has_zeros, uint32_t flags, char *buf, size_t buf_len);

#ifdef __cplusplus
}
#endif
#endif /* MATGPTQ_ABI_H */
