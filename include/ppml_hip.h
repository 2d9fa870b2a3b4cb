/*
 * ppml_hip.h -- C ABI of the MI355X (gfx950) matrix-multiplication backend.
 *
 * Every entry point is the twin of one of the reference's per-op launcher functions (free
 * functions in namespace ppml, declared extern in src/backend/CUDAKernels.cpp:158-205 and
 * 325-326).  Arguments keep the reference's names, order and meaning; two things differ on
 * purpose: each launcher returns an int status instead of void (the reference's cudaCheck has an
 * empty body, src/cuda/CUDAKernels.cu:21-24, so its launch errors are dropped), and each takes
 * a trailing stream (NULL = the default stream, which is what the reference always uses).
 *
 * All pointers are DEVICE pointers owned by the caller's buffers; the library neither frees nor
 * retains them.  Launchers are asynchronous on the given stream; call ppml_hip_synchronize()
 * (Backend::synchronize, include/ppml/Backend.h:557) before reading results on the host.
 *
 * Status codes shared by all entry points:
 *   0 ok   1 bad arguments   2 K not a multiple of 32   3 allocation failed
 *   5 unsupported weight type   6 kernel launch failed   7 no usable gfx950 device
 */
#ifndef PPML_HIP_H
#define PPML_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PPML_HIP_ABI_VERSION 1

typedef void *ppml_hip_stream_t; /* a hipStream_t, or NULL */

/* Weight storage handed to mul_mat_q8_hip; 0..2 are the reference's wtype values
 * (src/backend/CUDAKernels.cpp:769-770), 3 is this library's MFMA-fragment layout. */
enum {
    PPML_WTYPE_Q8_0 = 0,  /* interleaved 34-byte block_q8_0  (include/ppml/QuantBlocks.h:33-36) */
    PPML_WTYPE_Q8_1 = 1,  /* interleaved 36-byte block_q8_1  (include/ppml/QuantBlocks.h:38-41) */
    PPML_WTYPE_Q8_0R = 2, /* qs plane + d plane              (include/ppml/QuantBlocks.h:113-135) */
    PPML_WTYPE_Q8_0M = 3  /* MFMA-fragment order, made by q8_weight_pack_hip */
};

/* ---- library / device --------------------------------------------------------------------- */
int ppml_hip_abi_version(void);
/* Selects `device`, checks that it is a gfx950 part; replaces cudaSetDevice in
 * CUDABackend::graph_compute (src/backend/CUDABackend.cpp:708-712). */
int ppml_hip_init(int device);
/* Backend::synchronize (include/ppml/Backend.h:557). */
int ppml_hip_synchronize(void);
/* Text of the last failure on the calling thread ("" if none). */
const char *ppml_hip_last_error(void);

/* ---- f32 GEMM ------------------------------------------------------------------------------ */
/* Which matrix pipe multiplies binary32 operands in the f32 contractions below: 0 (default) = the bf16 pipe
 * through an exact three-way split of every operand (binary32-grade results, about 1.5 times the speed),
 * 1 = the fp32 pipe (v_mfma_f32_32x32x2_f32, k ascending two at a time).  The environment variable
 * PPML_HIP_F32_ARITH=fp32 selects 1 before the first call.  Returns the previous setting; other values of
 * `mode` only query.  The setting belongs to the calling thread (threads that want different arithmetic do
 * not disturb each other; a new thread starts from the environment's choice).  No counterpart in the reference (its tf32 switch PPML_MUL_MAT_TC trades accuracy,
 * this one does not). */
int ppml_hip_set_f32_arithmetic(int mode);
/* replaces mul_mat_cuda (src/cuda/CUDAKernels.cu:1174-1182):
 * C[m*N+n] = (bias ? bias[n] : 0) + sum_k A[m*K+k] * B[n*K+k].  bias may be NULL.
 * Arithmetic of this and the other f32 contractions below: each binary32 operand is the exact sum of
 * three bf16 numbers; six of the nine partial products (all but 2^-23 of |a||b|) are formed exactly on
 * the bf16 matrix pipe and summed in binary32.  Two kinds of operand fall outside what three bf16 parts
 * carry: a non-finite one, and one with bits below 2^-133, bf16's smallest step (subnormal operands and the
 * smallest normal ones).  The kernels notice both while they split the operands and redo the outputs of the
 * affected tile in plain binary32 arithmetic, one product at a time with k ascending (the reference's own
 * loop): +-inf, NaN and the bits down to 2^-149 come out as the reference's.  The fused attention kernels
 * (flash_attn_*_hip) split without that check; ppml_hip_set_f32_arithmetic(1) selects the fp32 pipe, which
 * carries every operand, for all of them.  Contractions of at
 * least 512 work-groups of 256 x 128 outputs (6 bytes per operand element) and contractions of few output
 * tiles under a long K (the partial sums of their K slices) use a workspace from a stream-ordered pool of
 * the library's; a stream keeps one such buffer between calls (the per-thread default stream allocates and
 * releases per call).  A stream under capture gets no workspace -- an allocation made while a graph is recorded
 * is gone before the graph runs -- and its calls take the forms that need none; mul_mat_tn_noalloc_hip brings the
 * sliced forms to recorded code. */
int mul_mat_hip(const float *A, const float *B, float *C, int M, int K, int N,
                const float *bias, ppml_hip_stream_t stream);

/* replaces mul_mat_cuda_f16 / mul_mat_mma_f16(_smem) (src/cuda/CUDAKernels.cu:1186-1492, declared
 * src/backend/CUDAKernels.cpp:182-200): A and B hold IEEE halves, [M][K] and [N][K]; every product and the sum
 * are binary32 (a product of two halves is exact in binary32), C is f32.  bias may be NULL; it is added to
 * the finished sum, as the CPU kernel does on this branch (src/backend/CPUKernels.cpp:646-672). */
int mul_mat_f16_hip(const void *A16, const void *B16, float *C, int M, int K, int N,
                    const float *bias, ppml_hip_stream_t stream);

/* ---- Q8_0 ---------------------------------------------------------------------------------- */
/* Q8_0 twin of quantize_rows_q8_1_cuda (src/cuda/QuantKernels.cu:86-93); the arithmetic is
 * quantize_q8_0_host (include/ppml/QuantBlocks.h:62-79).  y receives ne/32 block_q8_0 records. */
int quantize_rows_q8_0_hip(const float *x, void *y, int64_t ne, ppml_hip_stream_t stream);
/* replaces dequantize_q8_0_cuda (src/cuda/QuantKernels.cu:95-101). */
int dequantize_q8_0_hip(const void *x, float *y, int64_t ne, ppml_hip_stream_t stream);
/* replaces quantize_rows_q8_1_cuda (src/cuda/QuantKernels.cu:86-93), the activation quantizer of the
 * reference's CUDA path: d = vmax / -128 with vmax the signed element of largest magnitude (first one
 * on equal magnitudes, as the host loop include/ppml/QuantBlocks.h:81-111 picks it), quants clamped to
 * [-128, 127], s = d * sum(quants).  y receives ne/32 block_q8_1 records (36 bytes). */
int quantize_rows_q8_1_hip(const float *x, void *y, int64_t ne, ppml_hip_stream_t stream);
/* replaces dequantize_q8_1_cuda (src/cuda/QuantKernels.cu:103-109). */
int dequantize_q8_1_hip(const void *x, float *y, int64_t ne, ppml_hip_stream_t stream);

/* Once-per-weight repack, the role repack_q8_0_host plays in the reference
 * (include/ppml/QuantBlocks.h:123-133, called from src/model/PPML.cpp:4504-4528).
 * Turns an M x K weight of type 0, 1 or 2 into PPML_WTYPE_Q8_0M. */
size_t q8_weight_packed_bytes_hip(int M, int K);
int q8_weight_pack_hip(const void *W, int wtype, int M, int K, void *packed,
                       ppml_hip_stream_t stream);

/* replaces mul_mat_q8_cuda (src/cuda/MulMatQ8Kernel.cu:476-547).
 * W: M x K quantized weight (rows = out features), X: N x K f32 activations (rows = tokens).
 * Activations are quantized to Q8_0 per 32-element block inside the kernel, every block is
 * contracted with int8 MFMA into an exact int32 and settled as
 *     acc = fma(float(sumi), d_w * d_a, acc)        blocks ascending
 * (src/cuda/MulMatQ8Kernel.cu:120-142).  c_trans 0 -> C[m*N+n], 1 -> C[n*M+m].
 * *path_out (may be NULL) receives what the reference would report for the call (MulMatQ8Kernel.cu:493-496):
 * 1 when PPML_MMQ is not 0 and N reaches PPML_MMQ_MIN_N (default 16) or the weight is repacked (wtype 2, 3),
 * else 0; 0 on every error.  It names the reference's kernels, not this library's (ppml_hip_q8_last_path
 * does that): every path gives the same numbers.
 * A packed weight (wtype 3) too large for the weight-stationary kernels, under enough tokens and features for
 * sixteen tiles of 128 x 256 (or 128 x 128), takes the tiled kernel: the activations are quantized once into a workspace
 * (1.06 bytes per element, fragment order) from the stream-ordered pool mul_mat_hip describes -- the only
 * kernel family of this entry point that uses memory beyond its arguments; without a workspace the general
 * kernel serves the call.  A weight of wtype 0, 1 or 2 beyond 256 Ki elements takes it too, packed into the same
 * workspace on the way (1.06 bytes per element more); a smaller one is packed into the workspace per call as well
 * (one launch, 3.7 us) and served by the kernels of wtype 3, where they have an instance and the call is large enough
 * for that launch to pay (2^27 products; 64 Ki weight elements with K >= 512 or 768 features at any token count). */
int mul_mat_q8_hip(const void *W, const float *X, float *C, int M, int N, int K, int wtype,
                   int c_trans, int *path_out, ppml_hip_stream_t stream);

/* The same kernel with its optional inputs and outputs exposed.
 *   flags bit 0: apply ReLU to X before quantizing (FeedForward: linear1 -> ReLU -> linear2,
 *                src/modules/Attention.cpp:1097-1104)
 *   flags bit 1: quantize X with the Q8_1 rule of quantize_rows_q8_1_hip instead of the Q8_0 rule:
 *                the numbers mul_mat_q8_cuda itself produces (src/cuda/MulMatQ8Kernel.cu:520-527
 *                quantizes activations to Q8_1 and settles with their d).
 *   flags bits 2..8 (PPML_Q8_FLAG_*): restrict the choice among the kernels that serve a Q8_0M weight (and a weight
 *                of another layout that is packed per call, below), all of which give the same bits; for tests and
 *                measurements.  (With c_trans = 0 the choice is
 *                between the weight-stationary kernel without column parts and the general one.)
 *   xq_dump  (may be NULL): receives the Q8_0 blocks the kernel made of X, [N][K/32] block_q8_0
 *   sums_dump(may be NULL): receives the per-block int32 sums, [(n*M+m)*(K/32)+ib]            */
enum {
    PPML_Q8_FLAG_RELU = 1,
    PPML_Q8_FLAG_Q8_1_ACTIVATIONS = 2,
    PPML_Q8_FLAG_NO_LOW_LATENCY = 4,       /* do not take the low-latency kernel */
    PPML_Q8_FLAG_NO_WEIGHT_STATIONARY = 8, /* do not take the weight-stationary kernel */
    PPML_Q8_FLAG_LOW_LATENCY_8 = 16,       /* low-latency kernel with units of 8 tokens wherever it has an instance */
    PPML_Q8_FLAG_LOW_LATENCY_16 = 32,      /* ... of 16 tokens */
    PPML_Q8_FLAG_LOW_LATENCY_32 = 48,      /* ... of 32 tokens (both bits; K = 512 only) */
    PPML_Q8_FLAG_COLUMN_PARTS = 64,        /* weight-stationary kernel: work-groups share a token tile, a part of the columns each, wherever there is an instance */
    PPML_Q8_FLAG_NO_COLUMN_PARTS = 128,    /* ... never */
    PPML_Q8_FLAG_NO_TILED = 256            /* do not take the tiled kernel (large weights under many tokens) */
};
int mul_mat_q8_ex_hip(const void *W, const float *X, float *C, int M, int N, int K, int wtype,
                      int c_trans, int flags, void *xq_dump, int32_t *sums_dump,
                      ppml_hip_stream_t stream);

/* ---- batched / permuted f32 contractions ----------------------------------------------------- */
/* replaces out_prod_cuda (src/cuda/OutProdKernel.cu:211-260) with the CPU kernel's plane
 * broadcast (src/backend/CPUKernels.cpp:836-858):
 * dst[i0,i1,i2,i3] = sum_k src0[i0,k,i2/(ne2/ne02),i3/(ne3/ne03)] * src1[i1,k,i2,i3].
 * dst is overwritten (the caller does not need to zero it first). */
int out_prod_hip(const float *src0, const float *src1, float *dst,
                 int64_t ne00, int64_t ne01, int64_t ne02, int64_t ne03,
                 int64_t ne10, int64_t ne11, int64_t ne12, int64_t ne13,
                 int64_t ne0, int64_t ne1, int64_t ne2, int64_t ne3,
                 ppml_hip_stream_t stream);
/* out_prod_hip of the {1,0,2,3} permutations of both operands, without the permutation copies -- the second
 * contraction of the attention chain as the reference builds it, out_prod(permute(attn), permute(V))
 * (src/modules/Attention.cpp:277-281; its permute is a copy, src/core/ComputeGraphHelper.cpp:700-729):
 * dst[i0,i1,i2,i3] = sum_k src0[k,i0,i2/(ne2/ne02),i3/(ne3/ne03)] * src1[k,i1,i2,i3], dimensions of the operands AS
 * THEY LIE (ne00 = ne10 = the contracted length, ne0 = ne01, ne1 = ne11).  Same kernel, same products in the same
 * order as out_prod_hip on the permuted copies: same bits.  No counterpart among the reference's launchers. */
int out_prod_tt_hip(const float *src0, const float *src1, float *dst,
                    int64_t ne00, int64_t ne01, int64_t ne02, int64_t ne03,
                    int64_t ne10, int64_t ne11, int64_t ne12, int64_t ne13,
                    int64_t ne0, int64_t ne1, int64_t ne2, int64_t ne3,
                    ppml_hip_stream_t stream);
/* out_prod followed by the OP_SCALE node of the attention path in one pass
 * (src/modules/Attention.cpp:264-270): dst = scale * out_prod(src0, src1). */
int out_prod_scaled_hip(const float *src0, const float *src1, float *dst,
                        int64_t ne00, int64_t ne01, int64_t ne02, int64_t ne03,
                        int64_t ne10, int64_t ne11, int64_t ne12, int64_t ne13,
                        int64_t ne0, int64_t ne1, int64_t ne2, int64_t ne3,
                        float scale, ppml_hip_stream_t stream);

/* replaces outer_prod_mean_cuda (src/cuda/PairKernels.cu:553-561), indexing of
 * src/backend/CPUKernels.cpp:1006-1028: left/right [D,L,N,B] -> dst [D*D,L,L,B]. */
int outer_prod_mean_hip(const float *left, const float *right, float *dst,
                        int64_t D, int64_t L, int64_t N, int64_t B, float inv_N,
                        ppml_hip_stream_t stream);
/* replaces outer_prod_mean_back_cuda (declared src/backend/CUDAKernels.cpp:327-330), mathematics of
 * CPUBackend::kernel_outer_prod_mean_back (src/backend/CPUKernels.cpp:1034-1105): grad [D*D,L,L,B], left and
 * right [D,L,N,B] -> gleft, gright [D,L,N,B] (either may be NULL, not both):
 *   gleft[d1,i,n,b]  = inv_N * sum_{j,d2} grad[(d1*D+d2),i,j,b] * right[d2,j,n,b]
 *   gright[d2,j,n,b] = inv_N * sum_{i,d1} grad[(d1*D+d2),i,j,b] * left[d1,i,n,b] */
int outer_prod_mean_back_hip(const float *grad, const float *left, const float *right, float *gleft, float *gright,
                             int64_t D, int64_t L, int64_t N, int64_t B, float inv_N, ppml_hip_stream_t stream);
/* value-form outer product mean (src/ops/MathUtils.cpp:387-437):
 * left/right (B,N,L,D) -> dst (B,L,L,D*D), i.e. dst = A^T B / N per batch. */
int outer_product_mean_value_hip(const float *left, const float *right, float *dst,
                                 int64_t B, int64_t N, int64_t L, int64_t D,
                                 ppml_hip_stream_t stream);
/* The plain form of the same contraction: O[m*Nc+n] = alpha * sum_k A[k*M+m] * Bm[k*Nc+n]. */
int mul_mat_tn_hip(const float *A, const float *Bm, float *O, int M, int K, int Nc, float alpha,
                   ppml_hip_stream_t stream);

/* mul_mat_tn_hip for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc): the same contraction with the same kernels and the same bits, but the workspace the
 * large cases need (the bf16 planes of both operands, 6 bytes per padded operand element, plus the partial sums
 * of K slices) is a static 64 MiB device array of the library instead of a pool allocation.  It has no
 * counterpart in the reference.  The call allocates and frees nothing and records no statistics.  A contraction
 * whose workspace exceeds 64 MiB is refused with status 1 and a message that names both sizes (for two square
 * operands without K slices that is (M_pad + N_pad) * K_pad * 6 bytes, M padded to 256, N to 128, K to 16:
 * e.g. 12288 x 256 x 12288 takes 36 MiB); contractions that need no workspace run whatever their size.  The
 * array's address on a device is looked up by ppml_hip_init(device) -- or by the first call on a device that
 * was never initialised, so call ppml_hip_init first where even that lookup is unwelcome.  All calls on one GPU
 * share that GPU's array: calls that overlap in time on one GPU (two streams, two threads) race; order them. */
int mul_mat_tn_noalloc_hip(const float *A, const float *Bm, float *O, int M, int K, int Nc, float alpha,
                           ppml_hip_stream_t stream);

/* replaces tri_mul_cuda (src/cuda/PairKernels.cu:514-523, declared src/backend/CUDAKernels.cpp:316-318),
 * indexing and finite guard of CPUBackend::kernel_tri_mul (src/backend/CPUKernels.cpp:907-968):
 *   outgoing: dst[((d*I+i)*J+j)*B+b] = inv_L * sum_k left[((d*I+i)*K+k)*B+b] * right[((d*J+j)*K+k)*B+b]
 *   incoming: dst[((d*I+i)*J+j)*B+b] = inv_L * sum_k left[((d*K+k)*I+i)*B+b] * right[((d*K+k)*J+j)*B+b]
 * then NaN -> 0 and values beyond +-1e4 -> +-1e4.  One fp32-MFMA contraction per (d, b) plane. */
int tri_mul_hip(const float *left, const float *right, float *dst,
                int64_t D, int64_t I, int64_t J, int64_t K, int64_t B, float inv_L, int outgoing,
                ppml_hip_stream_t stream);

/* replaces tri_mul_back_cuda (src/cuda/PairKernels.cu:525-560, declared src/backend/CUDAKernels.cpp:320-323),
 * mathematics of CPUBackend::kernel_tri_mul_back (src/backend/CPUKernels.cpp:1238-1367): the gradients of
 * tri_mul_hip's two operands, each 1/L times a contraction of grad [D,I,J,B] with the other operand; gleft or
 * gright may be NULL (skipped), not both.  No finite guard here, as in the reference. */
int tri_mul_back_hip(const float *grad, const float *left, const float *right, float *gleft, float *gright,
                     int64_t D, int64_t I, int64_t J, int64_t K, int64_t B, float inv_L, int outgoing,
                     ppml_hip_stream_t stream);

/* ---- fused attention forward ------------------------------------------------------------------ */
/* replaces flash_attn_forward_cuda (declared src/backend/CUDAKernels.cpp:174, contract
 * include/ppml/FlashAttn.h:8-65, called from kernel_flash_attn_ext_cuda, CUDAKernels.cpp:894-903);
 * the fields of FlashAttnConfig are passed one by one.  The mathematics is that of
 * flash_attn_forward_cpu (src/ops/FlashAttn.cpp:55-135):
 *     O = softmax(scale * Q K^T + bias) V,  LSE = m + log(l + softmax_eps),  O = acc / (l + softmax_eps)
 * Q, K, V, O: [B][h][L][d] f32, 16-byte aligned; bias (may be NULL): [B][h][L query][L key];
 * LSE (may be NULL): [B][h][L].  scale <= 0 means 1/sqrt(d).  causal: key j <= query i only.
 * Bc is the reference's key-block width (<= 0 means 64); it does not change the arithmetic except
 * for one corner the reference has: a row whose first Bc keys are all masked with -inf is written
 * as O = 0, LSE = -inf even if later keys are not masked, as is a row masked entirely.
 * returns 0 = ran; 1 = refused (null pointer, non-positive size, d > 64 or d % 4 != 0 -- the
 * rule of src/backend/CUDABackend.cpp:457-463 -- misaligned pointer, B*h > 65535); 6 = launch error. */
int flash_attn_forward_hip(int B, int h, int L, int d, int causal, float scale, float softmax_eps, int Bc,
                           const float *Q, const float *K, const float *V, const float *bias,
                           float *O, float *LSE, ppml_hip_stream_t stream);

/* The same computation on tensors that have not been through the layout bridges the reference's graph
 * builder puts around the fused node (src/core/ComputeGraphHelper.cpp:456-458, 483): layout bit 0 -- Q, K
 * and V are [B][h][d][L] (the graph's [L, D, h, B] tensors); bit 1 -- O is written as [B][h][d][L].  It lets an
 * executor skip those four permutation copies.  No counterpart in the reference. */
int flash_attn_forward_ex_hip(int B, int h, int L, int d, int causal, float scale, float softmax_eps, int Bc,
                              const float *Q, const float *K, const float *V, const float *bias,
                              float *O, float *LSE, int layout, ppml_hip_stream_t stream);

/* replaces flash_attn_backward_cuda (declared src/backend/CUDAKernels.cpp:176-179, contract
 * include/ppml/FlashAttn.h:67-101, called from kernel_flash_attn_back_cuda, CUDAKernels.cpp:905-924), the
 * mathematics of flash_attn_backward_cpu (src/ops/FlashAttn.cpp:140-210): from dO and the forward's O and LSE,
 *     P = exp(S - LSE),  D_i = sum_d dO_id O_id,  dS = P (dO V^T - D),
 *     dQ = scale dS K,   dK = scale dS^T Q,   dV = P^T dO,   dbias = dS  (0 at masked positions)
 * Layouts as in flash_attn_forward_hip; dQ, dK, dV, dbias may each be NULL (not all).  Every output element is
 * written (rows with LSE = -inf as zeros), nothing needs clearing beforehand, and there are no atomics: results
 * do not depend on scheduling.  d <= 64 and a multiple of 4 (the reference's CUDA path stops at 32).
 * returns 0 = ran, 1 = refused, 6 = launch error. */
int flash_attn_backward_hip(int B, int h, int L, int d, int causal, float scale,
                            const float *Q, const float *K, const float *V, const float *bias,
                            const float *O, const float *dO, const float *LSE,
                            float *dQ, float *dK, float *dV, float *dbias, ppml_hip_stream_t stream);

/* ---- dimension permutation (a real copy) ------------------------------------------------------ */
/* replaces permute_cuda and transpose_cuda (declared src/backend/CUDAKernels.cpp:137-143, called from
 * kernel_permute_cuda / kernel_transpose_cuda, 1344-1390); semantics of CPUBackend::kernel_permute
 * (src/backend/CPUKernels.cpp:1669-1717): dimension p of dst is dimension d_p of src, both dense with
 * dimension 0 innermost.  s0..s3 are the source sizes, dd0..dd3 the destination sizes, total their
 * product; entries past ndim are ignored.  This is what mat_transpose(), the operand shuffles of the
 * backward GEMMs and the layout bridges around the fused attention node are made of.
 * returns 0 ok, 1 bad arguments (axes that are no permutation -- the reference refuses those too,
 * CUDAKernels.cpp:1376-1381 -- or sizes that do not match them), 6 launch error. */
int permute_hip(const float *src, float *dst, int64_t total, int ndim,
                int32_t d0, int32_t d1, int32_t d2, int32_t d3,
                int64_t s0, int64_t s1, int64_t s2, int64_t s3,
                int64_t dd0, int64_t dd1, int64_t dd2, int64_t dd3, ppml_hip_stream_t stream);

/* ---- sum over the copies of a broadcast (the bias gradient of mul_mat) ------------------------- */
/* replaces repeat_back4_cuda (declared src/backend/CUDAKernels.cpp:336-339, called from
 * kernel_repeat_back_cross_cuda, 1290-1320); semantics of CPUBackend::kernel_repeat_back
 * (src/backend/CPUKernels.cpp:2091-2148):
 *   dst[j0,j1,j2,j3] = sum_{k0<r0, k1<r1, k2<r2, k3<r3} src[j0+k0*d0, j1+k1*d1, j2+k2*d2, j3+k3*d3]
 * s0..s3 source sizes, d0..d3 destination sizes (dimension 0 innermost), r0..r3 copies per dimension as the
 * caller derives them (integer quotient of the sizes, dimension d of dst against dimension d of src).  This
 * is the node the backward of a biased mul_mat emits for the bias: grad [N, M] -> dbias [N]
 * (src/core/ComputeGraph.cpp:742).  The reference adds the copies one at a time, k3 fastest; here that
 * sequence is cut into consecutive runs summed side by side and added in run order (a fixed bracketing,
 * no atomics).  With few destination elements and many copies the partial sums take the stream's workspace
 * (see mul_mat_hip).  returns 0 ok, 1 bad arguments (a copy outside the source), 6 launch error. */
int repeat_back_hip(const float *src, float *dst,
                    int64_t s0, int64_t s1, int64_t s2, int64_t s3,
                    int64_t d0, int64_t d1, int64_t d2, int64_t d3,
                    int64_t r0, int64_t r1, int64_t r2, int64_t r3, ppml_hip_stream_t stream);

/* ---- element-wise nodes between the contractions ------------------------------------------------ */
/* The nodes the reference's graphs put between two matrix multiplications, so that such a graph stays on the
 * device: FeedForward is linear -> relu -> linear (src/modules/Attention.cpp:1097-1104), the attention logits are
 * out_prod -> scale -> add(bias) -> softmax (Attention.cpp:264-273).  All are HBM-bound streaming kernels. */

/* replaces scale_cuda (declared src/backend/CUDAKernels.cpp:257, called from kernel_scale_cuda, 992-1004);
 * semantics of CPUBackend::kernel_scale (src/backend/CPUKernels.cpp:1737-1754): dst[i] = x[i] * scale.
 * returns 0 ok, 1 bad arguments, 6 launch error. */
int scale_hip(const float *x, float *dst, float scale, int64_t nelements, ppml_hip_stream_t stream);

/* replaces unary_cuda (declared src/backend/CUDAKernels.cpp:208, called from kernel_unary_cuda, 666-672; its
 * block_size argument is a launch detail and has no counterpart).  uop is the reference's unary_op value
 * (include/ppml/ComputeGraph.h:20-39); this backend serves UNARY_OP_RELU = 4, the one between the configured
 * matrix multiplications: dst[i] = src[i] > 0 ? src[i] : 0 (compute_forward_relu, src/backend/CPUKernels.cpp:
 * 2649-2657: NaN and -0 give +0).  returns 0 ok, 1 bad arguments or another uop, 6 launch error. */
int unary_hip(const float *src, float *dst, int64_t n, int uop, ppml_hip_stream_t stream);

/* replaces bcast_elemwise_cuda (declared src/backend/CUDAKernels.cpp:114-118, called from
 * kernel_elemwise_{add,sub,mul,div}_cuda, 678-712); semantics of CPUBackend::kernel_elemwise
 * (src/backend/CPUKernels.cpp:446-596): dst[i] = a[i % an] op b[i % bn] for i < n, eop 0 add, 1 sub, 2 mul,
 * 3 div (IEEE division) -- an operand shorter than dst repeats along dst's flat order, i.e. it covers dst's
 * innermost dimensions.  an and bn must divide n (the reference reads on through an operand that does not and
 * only warns, CPUKernels.cpp:507-514; here that is status 1).  returns 0 ok, 1 bad arguments, 6 launch error. */
int bcast_elemwise_hip(const float *a, const float *b, float *dst, int64_t n, int64_t an, int64_t bn, int eop,
                       ppml_hip_stream_t stream);

/* replaces softmax_cuda (declared src/backend/CUDAKernels.cpp:153, called from kernel_softmax_cuda, 849-857;
 * block_size dropped); semantics of CPUBackend::kernel_softmax (src/backend/CPUKernels.cpp:1446-1467): M rows of
 * N values, output[r][d] = exp(x[r][d] - max_r) * (1 / (sum_d exp(x[r][d] - max_r) + 1e-9)).  The maximum starts
 * from the row's first element and moves on `>` only (a NaN there makes the whole row NaN, as in the reference).
 * The sum is formed across a wavefront, not d ascending: results agree with the reference's to rounding
 * (a few units in the last place), not bit for bit.  returns 0 ok, 1 bad arguments, 6 launch error. */
int softmax_hip(const float *input, float *output, int M, int N, ppml_hip_stream_t stream);
/* softmax_hip on input + bias, without the sum going to memory: the OP_ADD node in front of the attention softmax
 * (src/modules/Attention.cpp:271-276) folded into it.  Row r of the input is added to row r % bias_rows of `bias`
 * ([bias_rows][N]; bias_rows must divide M: the flat-modulo rule of bcast_elemwise_hip for an operand of whole
 * rows), one binary32 addition per element exactly as the node makes it, so the result has the bits of
 * softmax_hip(bcast_elemwise_hip(input, bias, add)).  It has no counterpart among the reference's launchers (its
 * graphs run the two nodes).  returns 0 ok, 1 bad arguments, 6 launch error. */
int softmax_add_hip(const float *input, const float *bias, float *output, int M, int N, int bias_rows,
                    ppml_hip_stream_t stream);

/* ---- observability (include/ppml/MulMatStats.h:39-169, src/cuda/CUDAKernels.cu:1693-1732) ------ */
/* MUL_MAT statistics: per (path, M, K, N) the number of launcher calls and the device time of their
 * launches, measured with a pair of events recorded on the launcher's stream (nothing waits; inside a
 * stream capture only the call is counted).  Enabled by the environment variable PPML_MULMAT_STATS (set and
 * not "0", the reference's rule) or by ppml_hip_mulmat_stats_enable(1); while enabled, the table is also
 * printed to stderr when the process exits, as the reference does.  Shapes are kept whole (the reference's
 * key holds 20 bits per dimension). */
typedef struct ppml_hip_mulmat_stat {
    char path[32];   /* "hip/<kernel family>", the reference's "<where>/<path>" bucket name */
    int64_t M, K, N; /* output rows, contracted length, output columns, as the reference prints them */
    int64_t calls;
    double ms;       /* accumulated device time of the calls whose launches have finished */
} ppml_hip_mulmat_stat;
/* Switches the statistics on (1) or off (0); other values only query.  Returns the previous state. */
int ppml_hip_mulmat_stats_enable(int on);
/* Writes up to `cap` rows of {M, K, N, calls} (int64 each), summed over the paths, ordered by shape;
 * returns the number of distinct shapes. */
int ppml_hip_mulmat_stats(int64_t *rows, int cap);
/* Waits for the recorded launches, then writes up to `cap` rows ordered by (path, M, K, N); returns the
 * number of rows the table holds.  mulmat_stats_record's table (MulMatStats.h:154-169) read back. */
int ppml_hip_mulmat_stats_rows(ppml_hip_mulmat_stat *rows, int cap);
/* mulmat_stats_dump (MulMatStats.h:86-145): totals, per-path lines and the top 12 shapes, to stderr. */
void ppml_hip_mulmat_stats_dump(void);
/* Empties the table (recorded launches are waited for first). */
void ppml_hip_mulmat_stats_reset(void);

/* Which kernel family served the calling thread's last mul_mat_q8_hip / mul_mat_q8_ex_hip call: the
 * counterpart of mul_mat_q8_cuda's *path_out (src/cuda/MulMatQ8Kernel.cu:476, 1 = MMQ, 0 = MMVQ), whose
 * two values do not describe this library's kernels. */
enum {
    PPML_Q8_PATH_GENERAL = 0,           /* one token tile per work-group, any shape and weight layout */
    PPML_Q8_PATH_WEIGHT_STATIONARY = 1, /* persistent work-groups, weight fragments resident in registers */
    PPML_Q8_PATH_LOW_LATENCY = 2,       /* few token tiles per CU: many small work-groups, weights through L2 */
    PPML_Q8_PATH_TILED = 3              /* large weights under many tokens: activations quantized ahead, 128 x 256 tiles */
};
int ppml_hip_q8_last_path(void);

#ifdef __cplusplus
}
#endif
#endif
