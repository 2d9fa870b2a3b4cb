/*
 * ppml_oracle.h -- CPU restatement of the reference's matrix-multiplication path.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker for the HIP kernels: it is
 * loaded by the test-suite, by the smoke check and by the benchmark's cpu_baseline leg.
 * Nothing in the shipped GPU path may call it; the GPU library has no CPU fallback.
 *
 * Every function cites the reference file:line whose loop it restates
 * (paths relative to the reference tree).  Storage conventions are the reference's:
 *   block_q8_0  = { fp16 d; int8 qs[32]; }  34 bytes, 2-byte aligned   (include/ppml/QuantBlocks.h:33-36)
 *   Q8_0R       = qs plane [nblocks][32] followed by d plane [nblocks] fp16 (QuantBlocks.h:113-135)
 *
 * Pinning status of each function is recorded next to its definition in ppml_oracle.c.
 */
#ifndef PPML_ORACLE_H
#define PPML_ORACLE_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_QK8_0 32
#define ORC_Q8_0_BLOCK_BYTES 34

/* include/ppml/HalfUtils.h:26-52 */
uint16_t orc_fp32_to_fp16(float f);
float    orc_fp16_to_fp32(uint16_t h);

/* include/ppml/QuantBlocks.h:62-79 ; returns 0 on success, 1 if n % 32 != 0 */
int  orc_quantize_q8_0(const float *src, void *dst_blocks, int64_t n);
/* include/ppml/QuantBlocks.h:123-145 */
size_t orc_q8_0_repacked_bytes(int64_t numel);
void orc_repack_q8_0(const void *src_blocks, int64_t nblocks, void *dst);
void orc_unrepack_q8_0(const void *src, int64_t nblocks, void *dst_blocks);
/* include/ppml/QuantBlocks.h:164-170 */
void orc_dequantize_q8_0(const void *src_blocks, float *dst, int64_t n);

/* per-block int32 sums of src/cuda/MulMatQ8Kernel.cu:120-139:
 * sums[(n*M + m)*nblk + ib] = sum_{i<32} W[m][ib].qs[i] * X[n][ib].qs[i]      */
int  orc_q8_block_sums(const void *w_blocks, const void *x_blocks, int32_t *sums,
                       int M, int N, int K);

/* src/cuda/MulMatQ8Kernel.cu:108-145 on two Q8_0 operands (M = weight rows, N = activation rows).
 * c_trans 0: C[m*N+n]   c_trans 1: C[n*M+m].   fma != 0 -> acc = fmaf(float(sumi), dw*da, acc)
 * (what nvcc's default contraction makes of the reference line), fma == 0 -> rounded product
 * then rounded add.  returns 0 ok, 1 bad args, 2 K % 32.                                      */
int  orc_mul_mat_q8q8(const void *w_blocks, const void *x_blocks, float *C,
                      int M, int N, int K, int c_trans, int fma, int nthreads);
/* Whole Q8_0 linear: quantize every activation row with orc_quantize_q8_0, then the loop above.
 * wtype 0 = interleaved block_q8_0, 2 = Q8_0R; others -> 5 (src/cuda/MulMatQ8Kernel.cu:476-547). */
int  orc_mul_mat_q8(const void *W, const float *X, float *C, int M, int N, int K,
                    int wtype, int c_trans, int fma, int nthreads);

/* include/ppml/QuantBlocks.h:81-111: the activation quantizer of the reference's CUDA path;
 * dst receives n/32 block_q8_1 records {fp16 d; fp16 s; int8 qs[32]} (36 bytes). */
int  orc_quantize_q8_1(const float *src, void *dst_blocks, int64_t n);
/* orc_mul_mat_q8 with the activation rule selectable: act 0 = Q8_0 (CPU contract), 1 = Q8_1 (what
 * mul_mat_q8_cuda computes, src/cuda/MulMatQ8Kernel.cu:483-527). */
int  orc_mul_mat_q8_act(const void *W, const float *X, float *C, int M, int N, int K,
                        int wtype, int c_trans, int fma, int act, int nthreads);

/* src/backend/CPUKernels.cpp:763-771 ; bias may be NULL */
void orc_mul_mat_f32(const float *a, const float *b, float *d, int M, int K, int N,
                     const float *bias, int nthreads);
/* src/backend/CPUKernels.cpp:392-396, 646-672: halves in, binary32 products and sum, bias last */
void orc_mul_mat_f16(const uint16_t *a, const uint16_t *b, float *d, int M, int K, int N,
                     const float *bias, int nthreads);

/* src/backend/CPUKernels.cpp:787-887 */
void orc_out_prod(const float *s0, const float *s1, float *dst,
                  int64_t ne00, int64_t ne01, int64_t ne02, int64_t ne03,
                  int64_t ne10, int64_t ne11, int64_t ne12, int64_t ne13,
                  int64_t ne0, int64_t ne1, int64_t ne2, int64_t ne3, int nthreads);
/* src/backend/CPUKernels.cpp:982-1032 */
void orc_outer_prod_mean(const float *left, const float *right, float *dst,
                         int64_t D, int64_t L, int64_t N, int64_t B, int nthreads);
/* src/backend/CPUKernels.cpp:1034-1105 (kernel_outer_prod_mean_back); gleft / gright may be NULL */
void orc_outer_prod_mean_back(const float *grad, const float *left, const float *right, float *gleft, float *gright,
                              int64_t D, int64_t L, int64_t N, int64_t B, int nthreads);
/* src/ops/MathUtils.cpp:387-437 */
void orc_outer_product_mean_value(const float *left, const float *right, float *dst,
                                  int64_t B, int64_t N, int64_t L, int64_t D, int nthreads);
/* src/modules/Attention.cpp:58-79 (scores only, before bias and softmax) */
void orc_attention_scores(const float *Q, const float *K, float *scores,
                          int64_t NQ, int64_t H, int64_t D, int64_t Lq, int64_t Lk, int nthreads);

/* src/ops/FlashAttn.cpp:55-135 (flash_attn_forward_cpu): O = softmax(scale * Q K^T + bias) V, one pass over
 * key blocks of Bc with a running maximum and sum.  Q, K, V, O are [B][h][L][d], bias (may be NULL) is
 * [B][h][L query][L key], LSE (may be NULL) is [B][h][L].  scale <= 0 -> 1/sqrt(d).  A row whose sum
 * is 0 gets O = 0, LSE = -inf.  returns 0 ok, 1 bad arguments (null pointer, non-positive dimension). */
int orc_flash_attn_forward(int B, int h, int L, int d, int causal, float scale, float softmax_eps, int Bc,
                           const float *Q, const float *K, const float *V, const float *bias,
                           float *O, float *LSE, int nthreads);

/* src/backend/CPUKernels.cpp:907-968 (kernel_tri_mul): d outermost, b innermost in every tensor;
 * outgoing contracts left[d,i,k,b] right[d,j,k,b], incoming left[d,k,i,b] right[d,k,j,b]; result times
 * 1/L, then the finite guard (NaN -> 0, beyond +-1e4 -> +-1e4). */
void orc_tri_mul(const float *left, const float *right, float *dst,
                 int64_t D, int64_t I, int64_t J, int64_t K, int64_t B, float L, int outgoing, int nthreads);

/* src/backend/CPUKernels.cpp:1238-1367 (kernel_tri_mul_back): gleft has left's shape, gright right's;
 * either may be NULL here (the CPU kernel wants both, the CUDA wrapper accepts one). */
void orc_tri_mul_back(const float *grad, const float *left, const float *right, float *gleft, float *gright,
                      int64_t D, int64_t I, int64_t J, int64_t K, int64_t B, float L, int outgoing, int nthreads);

/* src/backend/CPUKernels.cpp:1669-1717 (kernel_permute): dimension p of dst is dimension axes[p] of src;
 * sd = source sizes, dd = destination sizes (dims[0] innermost), entries past ndim ignored.
 * returns 0 ok, 1 when an axis is outside [0, ndim) -- the reference prints and leaves dst untouched. */
int orc_permute(const float *src, float *dst, int ndim, const int32_t axes[4], const int64_t sd[4], const int64_t dd[4]);

/* src/ops/FlashAttn.cpp:140-210 (flash_attn_backward_cpu): gradients of orc_flash_attn_forward's inputs from
 * dO, with P = exp(S - LSE) recomputed.  dQ, dK, dV [B][h][L][d], dbias [B][h][L][L]; any of them may be NULL
 * (not all).  Outputs are zeroed first; rows with LSE = -inf and masked positions contribute nothing.
 * returns 0 ok, 1 bad arguments. */
int orc_flash_attn_backward(int B, int h, int L, int d, int causal, float scale,
                            const float *Q, const float *K, const float *V, const float *bias,
                            const float *O, const float *dO, const float *LSE,
                            float *dQ, float *dK, float *dV, float *dbias);

/* src/backend/CPUKernels.cpp:2091-2148 (kernel_repeat_back): dst = src summed over its copies; nd_* are the
 * ranks, sd / dd the sizes (dims[0] innermost), dimension d of dst meets dimension d of src. */
void orc_repeat_back(const float *src, float *dst, int nd_src, const int64_t sd[4], int nd_dst, const int64_t dd[4]);

/* The element-wise nodes between the contractions (one IEEE operation per element, so thread counts change
 * nothing): src/backend/CPUKernels.cpp:1737-1754 (kernel_scale), 2649-2657 (compute_forward_relu), 446-596
 * (kernel_elemwise: flat-modulo broadcast, eop 0 add 1 sub 2 mul 3 div), 1446-1467 (kernel_softmax over dims[0]). */
void orc_scale(const float *src, float *dst, int64_t n, float s, int nthreads);
void orc_relu(const float *src, float *dst, int64_t n, int nthreads);
int orc_bcast_elemwise(const float *a, const float *b, float *d, int64_t n, int64_t an, int64_t bn, int eop, int nthreads);
void orc_softmax(const float *src, float *dst, int64_t rows, int64_t D, int nthreads);

int orc_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif
