/*
 * ppml_oracle.c -- CPU restatement of the reference's matrix-multiplication path.
 *
 * TEST INFRASTRUCTURE ONLY (see ppml_oracle.h).  Build: `make -C oracle`
 * (gcc -O2 -ffp-contract=off -fopenmp; no fast-math, so every float operation rounds
 * exactly as the reference's x86-64 -O2 build, which has no FMA contraction).
 *
 * Pinning status (what fixes each function besides the reference text):
 *   orc_fp32_to_fp16 / orc_fp16_to_fp32 : own bit-level algorithm, checked against the
 *       reference's HalfUtils.h compiled as-is (oracle/_ref) and against numpy float16.
 *   orc_quantize_q8_0 : closed form per block; invariants (arg-max -> +-127, zero block ->
 *       d=0,q=0, |x - d*q| <= d/2), a hand-checked vector, and an independent
 *       double-precision restatement on random blocks.
 *   orc_repack/unrepack : round trip + plane offsets.
 *   orc_q8_block_sums   : exact integers, brute force with numpy int64.
 *   orc_mul_mat_q8q8    : PARITY UNPINNED by any reference-held test (the reference's own
 *       Q8 tests are absent from its tree and its CPU backend has no Q8 kernel); pinned
 *       by the closed form sum_ib float(sumi)*(dw*da) evaluated in float64 and by the
 *       dequantised f32 GEMM special case.
 *   orc_mul_mat_f32     : the reference's MulMat test inputs (tests/test_cuda.cpp:133-167),
 *       whose products and sums are exact in binary32, against integer arithmetic.
 *   orc_out_prod        : the reference's OutProd inputs (tests/test_cuda.cpp:207-245, 262-341),
 *       exact, plus broadcast special cases against numpy einsum.
 *   orc_outer_prod_mean : graph form; no reference-held vector covers its index decode and the
 *       reference kernel cannot be compiled here (CUDA headers absent) -- pinned only by numpy
 *       einsum over the layout stated at src/backend/CPUKernels.cpp:975-981.
 *   orc_outer_product_mean_value : known answers of tests/test_outer_product_mean.cpp:10-70.
 *   orc_attention_scores: einsum special case and the 1/sqrt(D) closed form.
 *   orc_tri_mul : numpy einsum over the layout stated at src/backend/CPUKernels.cpp:895-903 (outgoing and
 *       incoming), exact on small integers; the finite guard on planted NaN / Inf / 1e5 values.  No
 *       reference-held vector covers it.
 *   orc_outer_prod_mean_back : numpy einsum (exact on small integers) and the adjoint identity against
 *       orc_outer_prod_mean.
 *   orc_tri_mul_back : numpy einsum (exact on small integers) and the adjoint identity
 *       <grad, tri_mul(l, r)> = <gleft, l> = <gright, r> against orc_tri_mul, both forms.
 *   orc_permute : numpy.transpose with the axes translated (dst dim p = src dim axes[p], dims[0]
 *       innermost), identity and inverse permutations, hand-checked 2 x 3 case.
 *   orc_repeat_back : numpy sums over the broadcast axes on small integers (exact in any order), the
 *       bias-gradient case against a column sum, the mixed case where a dimension is both kept and
 *       repeated, the summation order probed with 2^24 + 1 + 1 (sequential from the left gives 2^24,
 *       any pairing of the two ones gives 2^24 + 2), and the dimension alignment of
 *       src/backend/CPUKernels.cpp:2099-2109 (dimension d of dst meets dimension d of src).
 *   orc_scale, orc_relu, orc_bcast_elemwise : one IEEE operation per element -- numpy's float32 operations
 *       bit for bit (np.float32 multiply, maximum-with-zero incl. NaN and -0 -> +0, add/sub/mul/div on
 *       np.resize'd operands, which is the flat-modulo broadcast); the prefix-broadcast case against numpy's
 *       own dimension-wise broadcasting.  No reference-held vector.
 *   orc_softmax : float64 softmax within 1e-6 (rows of equal values -> 1/(D + 1e-9 e^0 ...), i.e. the
 *       closed form 1 / (D + 1e-9) exactly where D is small; a dominant entry -> 1; shift invariance bit for
 *       bit for shifts that are exact; the 1e-9 in the denominator probed with a one-element row: 1/(1 + 1e-9)
 *       rounds to 1 in binary32 and exp(0) = 1, while a row of -inf gives NaN), and the composed chain
 *       scale -> add -> softmax -> second contraction against orc_flash_attn_forward on the golden vectors
 *       (tests/golden/flash_attn_forward.json).  No reference-held vector of the node itself.
 *   orc_flash_attn_forward : the reference's own src/ops/FlashAttn.cpp compiled as-is
 *       (oracle/_ref/libppml_ref_flash.so: it needs nothing but its header) -- bit-for-bit on
 *       random inputs, with and without bias, causal and not, ragged block sizes; plus float64
 *       softmax attention, closed forms (equal scores -> mean of V, one dominant key -> that
 *       row of V, shift invariance in the bias, fully masked rows) where the reference build
 *       is absent.
 *   orc_flash_attn_backward : the compiled reference routine bit for bit; central finite differences of
 *       the float64 softmax attention; rows of dbias sum to 0; masked rows give zero gradients.
 */
#include "ppml_oracle.h"

#include <math.h>
#include <string.h>
#include <stdlib.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static int pick_threads(int nthreads) {
#ifdef _OPENMP
    if (nthreads <= 0) return omp_get_max_threads();
    return nthreads;
#else
    (void)nthreads;
    return 1;
#endif
}

/* src/ops/FlashAttn.cpp:55-135.  Same loop nest, same order of the sums (dot product over d ascending,
 * scale, then bias; block maximum; alpha = exp(m - m_new) with 0 for the first block; P V per output
 * column over the block's keys ascending; acc = alpha * acc + pv; l = alpha * l + l_tile).  The planes
 * are independent, so they are spread over threads; within a row nothing is reordered. */
int orc_flash_attn_forward(int B, int h, int L, int d, int causal, float scale, float softmax_eps, int Bc,
                           const float *Q, const float *K, const float *V, const float *bias,
                           float *O, float *LSE, int nthreads) {
    if (!Q || !K || !V || !O) return 1;
    if (B <= 0 || h <= 0 || L <= 0 || d <= 0) return 1;
    if (Bc <= 0) Bc = 64;
    const float sc = scale > 0.0f ? scale : 1.0f / sqrtf((float)d);
    const int64_t planes = (int64_t)B * h;
    if (nthreads <= 0) nthreads = 1;
#pragma omp parallel for num_threads(nthreads) schedule(dynamic, 1)
    for (int64_t pl = 0; pl < planes; ++pl) {
        const float *Qb = Q + pl * (int64_t)L * d, *Kb = K + pl * (int64_t)L * d, *Vb = V + pl * (int64_t)L * d;
        float *Ob = O + pl * (int64_t)L * d;
        float *acc = (float *)malloc(sizeof(float) * (size_t)d);
        float *tile = (float *)malloc(sizeof(float) * (size_t)Bc);
        for (int i = 0; i < L; ++i) {
            const float *q = Qb + (int64_t)i * d;
            const int jmax = causal ? i + 1 : L;
            float m = -INFINITY, l = 0.0f;
            for (int dd = 0; dd < d; ++dd) acc[dd] = 0.0f;
            for (int j0 = 0; j0 < jmax; j0 += Bc) {
                const int j1 = j0 + Bc < jmax ? j0 + Bc : jmax, nb = j1 - j0;
                float m_tile = -INFINITY;
                for (int j = j0; j < j1; ++j) {
                    const float *k = Kb + (int64_t)j * d;
                    float s = 0.0f;
                    for (int dd = 0; dd < d; ++dd) s += q[dd] * k[dd];
                    s *= sc;
                    if (bias) s += bias[(pl * L + i) * (int64_t)L + j];
                    tile[j - j0] = s;
                    if (s > m_tile) m_tile = s;
                }
                const float m_new = m > m_tile ? m : m_tile;
                const float alpha = (m == -INFINITY) ? 0.0f : expf(m - m_new);
                float l_tile = 0.0f;
                for (int j = 0; j < nb; ++j) {
                    const float p = expf(tile[j] - m_new);
                    tile[j] = p;
                    l_tile += p;
                }
                for (int dd = 0; dd < d; ++dd) {
                    float pv = 0.0f;
                    for (int j = 0; j < nb; ++j) pv += tile[j] * Vb[(int64_t)(j0 + j) * d + dd];
                    acc[dd] = alpha * acc[dd] + pv;
                }
                l = alpha * l + l_tile;
                m = m_new;
            }
            float *o = Ob + (int64_t)i * d;
            if (l > 0.0f) {
                const float inv = 1.0f / (l + softmax_eps);
                for (int dd = 0; dd < d; ++dd) o[dd] = acc[dd] * inv;
                if (LSE) LSE[pl * L + i] = m + logf(l + softmax_eps);
            } else {
                for (int dd = 0; dd < d; ++dd) o[dd] = 0.0f;
                if (LSE) LSE[pl * L + i] = -INFINITY;
            }
        }
        free(acc);
        free(tile);
    }
    return 0;
}

/* src/backend/CPUKernels.cpp:1034-1105: per output one sequential binary32 sum, outer loop over the residue
 * index (j for gleft, i for gright), inner loop over the feature index, then times 1/N. */
void orc_outer_prod_mean_back(const float *grad, const float *left, const float *right, float *gleft, float *gright,
                              int64_t D, int64_t L, int64_t N, int64_t B, int nthreads) {
    const float inv_N = 1.0f / (float)N;
    const int64_t total = D * L * N * B;
    if (nthreads <= 0) nthreads = 1;
    if (gleft) {
#pragma omp parallel for num_threads(nthreads) schedule(static)
        for (int64_t idx = 0; idx < total; ++idx) {
            int64_t tmp = idx;
            const int64_t b = tmp % B; tmp /= B;
            const int64_t n = tmp % N; tmp /= N;
            const int64_t i = tmp % L;
            const int64_t d1 = tmp / L;
            float sum = 0.0f;
            for (int64_t j = 0; j < L; ++j)
                for (int64_t d2 = 0; d2 < D; ++d2)
                    sum += grad[(((d1 * D + d2) * L + i) * L + j) * B + b] * right[((d2 * L + j) * N + n) * B + b];
            gleft[idx] = sum * inv_N;
        }
    }
    if (gright) {
#pragma omp parallel for num_threads(nthreads) schedule(static)
        for (int64_t idx = 0; idx < total; ++idx) {
            int64_t tmp = idx;
            const int64_t b = tmp % B; tmp /= B;
            const int64_t n = tmp % N; tmp /= N;
            const int64_t j = tmp % L;
            const int64_t d2 = tmp / L;
            float sum = 0.0f;
            for (int64_t i = 0; i < L; ++i)
                for (int64_t d1 = 0; d1 < D; ++d1)
                    sum += grad[(((d1 * D + d2) * L + i) * L + j) * B + b] * left[((d1 * L + i) * N + n) * B + b];
            gright[idx] = sum * inv_N;
        }
    }
}

/* src/backend/CPUKernels.cpp:907-968: one output per index, k ascending, sequential binary32 sum. */
void orc_tri_mul(const float *left, const float *right, float *dst,
                 int64_t D, int64_t I, int64_t J, int64_t K, int64_t B, float L, int outgoing, int nthreads) {
    const float inv_L = 1.0f / L;
    const int64_t total = B * I * J * D;
    if (nthreads <= 0) nthreads = 1;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int64_t idx = 0; idx < total; ++idx) {
        int64_t tmp = idx;
        const int64_t b = tmp % B; tmp /= B;
        const int64_t j = tmp % J; tmp /= J;
        const int64_t i = tmp % I;
        const int64_t d = tmp / I;
        float sum = 0.0f;
        if (outgoing) {
            for (int64_t k = 0; k < K; ++k) sum += left[((d * I + i) * K + k) * B + b] * right[((d * J + j) * K + k) * B + b];
        } else {
            for (int64_t k = 0; k < K; ++k) sum += left[((d * K + k) * I + i) * B + b] * right[((d * K + k) * J + j) * B + b];
        }
        float v = sum * inv_L;
        if (!(v == v) || v > 1e4f || v < -1e4f) v = (v != v) ? 0.0f : (v > 1e4f ? 1e4f : -1e4f);
        dst[idx] = v;
    }
}

/* src/backend/CPUKernels.cpp:1238-1367: four index decodes, each output one sequential binary32 sum
 * (j ascending for gleft, i ascending for gright) times 1/L. */
void orc_tri_mul_back(const float *grad, const float *left, const float *right, float *gleft, float *gright,
                      int64_t D, int64_t I, int64_t J, int64_t K, int64_t B, float L, int outgoing, int nthreads) {
    const float inv_L = 1.0f / L;
    if (nthreads <= 0) nthreads = 1;
    if (gleft) {
        const int64_t total = D * I * K * B;
#pragma omp parallel for num_threads(nthreads) schedule(static)
        for (int64_t idx = 0; idx < total; ++idx) {
            int64_t tmp = idx, i, k, d;
            const int64_t b = tmp % B; tmp /= B;
            if (outgoing) { k = tmp % K; tmp /= K; i = tmp % I; d = tmp / I; }      /* gleft [d,i,k,b] */
            else          { i = tmp % I; tmp /= I; k = tmp % K; d = tmp / K; }      /* gleft [d,k,i,b] */
            float sum = 0.0f;
            for (int64_t j = 0; j < J; ++j) {
                const float gv = grad[((d * I + i) * J + j) * B + b];
                const float rv = outgoing ? right[((d * J + j) * K + k) * B + b] : right[((d * K + k) * J + j) * B + b];
                sum += gv * rv;
            }
            gleft[idx] = sum * inv_L;
        }
    }
    if (gright) {
        const int64_t total = D * J * K * B;
#pragma omp parallel for num_threads(nthreads) schedule(static)
        for (int64_t idx = 0; idx < total; ++idx) {
            int64_t tmp = idx, j, k, d;
            const int64_t b = tmp % B; tmp /= B;
            if (outgoing) { k = tmp % K; tmp /= K; j = tmp % J; d = tmp / J; }      /* gright [d,j,k,b] */
            else          { j = tmp % J; tmp /= J; k = tmp % K; d = tmp / K; }      /* gright [d,k,j,b] */
            float sum = 0.0f;
            for (int64_t i = 0; i < I; ++i) {
                const float gv = grad[((d * I + i) * J + j) * B + b];
                const float lv = outgoing ? left[((d * I + i) * K + k) * B + b] : left[((d * K + k) * I + i) * B + b];
                sum += gv * lv;
            }
            gright[idx] = sum * inv_L;
        }
    }
}

/* src/backend/CPUKernels.cpp:1669-1717: for every destination element, in order, decode its
 * coordinates (dims[0] innermost), place coordinate p at source dimension axes[p], read that element. */
int orc_permute(const float *src, float *dst, int ndim, const int32_t axes[4], const int64_t sd_in[4], const int64_t dd_in[4]) {
    int dims[4] = {0, 1, 2, 3};
    int64_t sd[4] = {1, 1, 1, 1}, dd[4] = {1, 1, 1, 1};
    for (int i = 0; i < ndim && i < 4; ++i) {
        dims[i] = axes[i];
        if (dims[i] < 0 || dims[i] >= ndim) return 1;
        sd[i] = sd_in[i];
        dd[i] = dd_in[i];
    }
    const int64_t total = dd[0] * dd[1] * dd[2] * dd[3];
    for (int64_t idx = 0; idx < total; ++idx) {
        int64_t t = idx;
        int64_t jv[4];
        jv[0] = t % dd[0]; t /= dd[0];
        jv[1] = t % dd[1]; t /= dd[1];
        jv[2] = t % dd[2]; t /= dd[2];
        jv[3] = t;
        int64_t i[4] = {0, 0, 0, 0};
        for (int p = 0; p < ndim && p < 4; ++p) i[dims[p]] = jv[p];
        dst[idx] = src[((i[3] * sd[2] + i[2]) * sd[1] + i[1]) * sd[0] + i[0]];
    }
    return 0;
}

/* src/ops/FlashAttn.cpp:140-210, same loop nest: rows i ascending, keys j ascending, every accumulation in
 * that order (dK and dV rows therefore receive their terms in ascending i).  Planes run on threads; nothing
 * inside a plane is reordered. */
int orc_flash_attn_backward(int B, int h, int L, int d, int causal, float scale,
                            const float *Q, const float *K, const float *V, const float *bias,
                            const float *O, const float *dO, const float *LSE,
                            float *dQ, float *dK, float *dV, float *dbias) {
    if (!Q || !K || !V || !O || !dO || !LSE) return 1;
    if (B <= 0 || h <= 0 || L <= 0 || d <= 0) return 1;
    if (!dQ && !dK && !dV && !dbias) return 1;
    const float sc = scale > 0.0f ? scale : 1.0f / sqrtf((float)d);
    const int64_t planes = (int64_t)B * h, nq = planes * L * d, nb = planes * L * L;
    if (dQ) memset(dQ, 0, sizeof(float) * (size_t)nq);
    if (dK) memset(dK, 0, sizeof(float) * (size_t)nq);
    if (dV) memset(dV, 0, sizeof(float) * (size_t)nq);
    if (dbias) memset(dbias, 0, sizeof(float) * (size_t)nb);
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t pl = 0; pl < planes; ++pl) {
        const int64_t po = pl * (int64_t)L * d;
        for (int i = 0; i < L; ++i) {
            const float lse = LSE[pl * L + i];
            if (!(lse > -INFINITY)) continue;
            const float *q = Q + po + (int64_t)i * d, *o_row = O + po + (int64_t)i * d, *do_row = dO + po + (int64_t)i * d;
            float Dsum = 0.0f;
            for (int dd = 0; dd < d; ++dd) Dsum += do_row[dd] * o_row[dd];
            const int jmax = causal ? i + 1 : L;
            for (int j = 0; j < jmax; ++j) {
                const float *k = K + po + (int64_t)j * d;
                float s = 0.0f;
                for (int dd = 0; dd < d; ++dd) s += q[dd] * k[dd];
                s *= sc;
                if (bias) s += bias[(pl * L + i) * (int64_t)L + j];
                const float p = expf(s - lse);
                float dp = 0.0f;
                for (int dd = 0; dd < d; ++dd) dp += do_row[dd] * V[po + (int64_t)j * d + dd];
                const float ds = p * (dp - Dsum);
                if (dbias) dbias[(pl * L + i) * (int64_t)L + j] = ds;
                if (dQ) for (int dd = 0; dd < d; ++dd) dQ[po + (int64_t)i * d + dd] += sc * ds * k[dd];
                if (dK) for (int dd = 0; dd < d; ++dd) dK[po + (int64_t)j * d + dd] += sc * ds * q[dd];
                if (dV) for (int dd = 0; dd < d; ++dd) dV[po + (int64_t)j * d + dd] += p * do_row[dd];
            }
        }
    }
    return 0;
}

int orc_max_threads(void) { return pick_threads(0); }

/* ------------------------------------------------------------------ fp16 */
/* Same function as include/ppml/HalfUtils.h:42-52 (round to nearest even, NaN -> sign|0x7E00),
 * written as explicit exponent/mantissa arithmetic rather than the reference's float-add trick. */
uint16_t orc_fp32_to_fp16(float f) {
    uint32_t u;
    memcpy(&u, &f, sizeof u);
    const uint32_t sign = (u >> 16) & 0x8000u;
    const uint32_t mag = u & 0x7fffffffu;
    if (mag > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);           /* NaN */
    if (mag >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);          /* >= 65520 -> inf */
    if (mag < 0x38800000u) {                                            /* below 2^-14: subnormal half */
        if (mag < 0x33000000u) return (uint16_t)sign;                   /* < 2^-25 -> 0 */
        const int e = (int)(mag >> 23);                                 /* biased exponent, 102..112 */
        const uint32_t m = (mag & 0x7fffffu) | 0x800000u;               /* 24-bit significand */
        const int shift = 126 - e;                                      /* result = m >> shift, 14..24 */
        uint32_t h = m >> shift;
        const uint32_t rem = m & ((1u << shift) - 1u);
        const uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (h & 1u))) h++;
        return (uint16_t)(sign | h);
    }
    uint32_t h = (((mag >> 23) - 112u) << 10) | ((mag & 0x7fffffu) >> 13);
    const uint32_t rem = mag & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;             /* carry may bump the exponent */
    return (uint16_t)(sign | h);
}

/* include/ppml/HalfUtils.h:26-37 (exact widening) */
float orc_fp16_to_fp32(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1fu;
    uint32_t m = h & 0x3ffu;
    uint32_t u;
    if (e == 0x1fu) {
        u = sign | 0x7f800000u | (m << 13);
    } else if (e != 0) {
        u = sign | ((e + 112u) << 23) | (m << 13);
    } else if (m == 0) {
        u = sign;
    } else {
        int ee = 113;
        while (!(m & 0x400u)) { m <<= 1; ee--; }
        u = sign | ((uint32_t)ee << 23) | ((m & 0x3ffu) << 13);
    }
    float f;
    memcpy(&f, &u, sizeof f);
    return f;
}

/* ------------------------------------------------------------------ Q8_0 */
static inline uint16_t blk_d_bits(const uint8_t *blk) {
    uint16_t d;
    memcpy(&d, blk, 2);
    return d;
}

/* include/ppml/QuantBlocks.h:62-79 */
int orc_quantize_q8_0(const float *src, void *dst_blocks, int64_t n) {
    if (n % ORC_QK8_0 != 0) return 1;
    const int64_t nb = n / ORC_QK8_0;
    uint8_t *out = (uint8_t *)dst_blocks;
    for (int64_t b = 0; b < nb; ++b) {
        const float *x = src + b * ORC_QK8_0;
        float amax = 0.0f;
        for (int i = 0; i < ORC_QK8_0; ++i) amax = fmaxf(amax, fabsf(x[i]));
        const float d = amax / 127.0f;
        const float inv = (amax == 0.0f) ? 0.0f : 1.0f / d;   /* the f32 d, not its fp16 rounding */
        const uint16_t dh = orc_fp32_to_fp16(d);
        uint8_t *blk = out + b * ORC_Q8_0_BLOCK_BYTES;
        memcpy(blk, &dh, 2);
        for (int i = 0; i < ORC_QK8_0; ++i) {
            float q = roundf(x[i] * inv);                     /* half away from zero */
            q = q > 127.0f ? 127.0f : (q < -127.0f ? -127.0f : q);
            ((int8_t *)(blk + 2))[i] = (int8_t)q;
        }
    }
    return 0;
}

/* include/ppml/QuantBlocks.h:119-121 */
size_t orc_q8_0_repacked_bytes(int64_t numel) {
    return (size_t)(numel / ORC_QK8_0) * (ORC_QK8_0 + 2);
}

/* include/ppml/QuantBlocks.h:123-133 */
void orc_repack_q8_0(const void *src_blocks, int64_t nblocks, void *dst) {
    const uint8_t *src = (const uint8_t *)src_blocks;
    uint8_t *qs = (uint8_t *)dst;
    uint8_t *d = qs + nblocks * ORC_QK8_0;
    for (int64_t b = 0; b < nblocks; ++b) {
        memcpy(qs + b * ORC_QK8_0, src + b * ORC_Q8_0_BLOCK_BYTES + 2, ORC_QK8_0);
        memcpy(d + b * 2, src + b * ORC_Q8_0_BLOCK_BYTES, 2);
    }
}

/* include/ppml/QuantBlocks.h:136-145 */
void orc_unrepack_q8_0(const void *src, int64_t nblocks, void *dst_blocks) {
    const uint8_t *qs = (const uint8_t *)src;
    const uint8_t *d = qs + nblocks * ORC_QK8_0;
    uint8_t *dst = (uint8_t *)dst_blocks;
    for (int64_t b = 0; b < nblocks; ++b) {
        memcpy(dst + b * ORC_Q8_0_BLOCK_BYTES + 2, qs + b * ORC_QK8_0, ORC_QK8_0);
        memcpy(dst + b * ORC_Q8_0_BLOCK_BYTES, d + b * 2, 2);
    }
}

/* include/ppml/QuantBlocks.h:164-170 */
void orc_dequantize_q8_0(const void *src_blocks, float *dst, int64_t n) {
    const uint8_t *src = (const uint8_t *)src_blocks;
    const int64_t nb = n / ORC_QK8_0;
    for (int64_t b = 0; b < nb; ++b) {
        const uint8_t *blk = src + b * ORC_Q8_0_BLOCK_BYTES;
        const float d = orc_fp16_to_fp32(blk_d_bits(blk));
        const int8_t *q = (const int8_t *)(blk + 2);
        for (int i = 0; i < ORC_QK8_0; ++i) dst[b * ORC_QK8_0 + i] = d * (float)q[i];
    }
}

static inline int32_t block_dot(const uint8_t *wb, const uint8_t *xb) {
    const int8_t *w = (const int8_t *)(wb + 2);
    const int8_t *x = (const int8_t *)(xb + 2);
    int32_t s = 0;
    for (int i = 0; i < ORC_QK8_0; ++i) s += (int32_t)w[i] * (int32_t)x[i];
    return s;
}

/* the integer part of src/cuda/MulMatQ8Kernel.cu:120-139 */
int orc_q8_block_sums(const void *w_blocks, const void *x_blocks, int32_t *sums,
                      int M, int N, int K) {
    if (!w_blocks || !x_blocks || !sums || M <= 0 || N <= 0 || K <= 0) return 1;
    if (K % ORC_QK8_0) return 2;
    const int nblk = K / ORC_QK8_0;
    const uint8_t *W = (const uint8_t *)w_blocks;
    const uint8_t *X = (const uint8_t *)x_blocks;
    for (int n = 0; n < N; ++n)
        for (int m = 0; m < M; ++m)
            for (int ib = 0; ib < nblk; ++ib)
                sums[((int64_t)n * M + m) * nblk + ib] =
                    block_dot(W + ((int64_t)m * nblk + ib) * ORC_Q8_0_BLOCK_BYTES,
                              X + ((int64_t)n * nblk + ib) * ORC_Q8_0_BLOCK_BYTES);
    return 0;
}

/* src/cuda/MulMatQ8Kernel.cu:108-145: one output = blocks ascending,
 * acc += float(sumi) * (d_w * d_a); d_w*d_a is the exact f32 product of two halves. */
int orc_mul_mat_q8q8(const void *w_blocks, const void *x_blocks, float *C,
                     int M, int N, int K, int c_trans, int fma, int nthreads) {
    if (!w_blocks || !x_blocks || !C || M <= 0 || N <= 0 || K <= 0) return 1;
    if (K % ORC_QK8_0) return 2;
    const int nblk = K / ORC_QK8_0;
    const uint8_t *W = (const uint8_t *)w_blocks;
    const uint8_t *X = (const uint8_t *)x_blocks;
    const int nt = pick_threads(nthreads);
    (void)nt;
#pragma omp parallel for schedule(dynamic, 4) num_threads(nt)
    for (int n = 0; n < N; ++n) {
        const uint8_t *xrow = X + (int64_t)n * nblk * ORC_Q8_0_BLOCK_BYTES;
        for (int m = 0; m < M; ++m) {
            const uint8_t *wrow = W + (int64_t)m * nblk * ORC_Q8_0_BLOCK_BYTES;
            float acc = 0.0f;
            for (int ib = 0; ib < nblk; ++ib) {
                const uint8_t *wb = wrow + ib * ORC_Q8_0_BLOCK_BYTES;
                const uint8_t *xb = xrow + ib * ORC_Q8_0_BLOCK_BYTES;
                const int32_t sumi = block_dot(wb, xb);
                const float s = orc_fp16_to_fp32(blk_d_bits(wb)) * orc_fp16_to_fp32(blk_d_bits(xb));
                if (fma) {
                    acc = fmaf((float)sumi, s, acc);
                } else {
                    const float t = (float)sumi * s;
                    acc = acc + t;
                }
            }
            if (c_trans) C[(int64_t)n * M + m] = acc;
            else         C[(int64_t)m * N + n] = acc;
        }
    }
    return 0;
}

/* src/cuda/MulMatQ8Kernel.cu:476-547 with Q8_0 activations (QuantBlocks.h:62-79 per row). */
int orc_mul_mat_q8(const void *W, const float *X, float *C, int M, int N, int K,
                   int wtype, int c_trans, int fma, int nthreads) {
    if (!W || !X || !C || M <= 0 || N <= 0 || K <= 0) return 1;
    if (K % ORC_QK8_0) return 2;
    if (wtype != 0 && wtype != 2) return 5;
    const int64_t nblk = K / ORC_QK8_0;
    uint8_t *xq = (uint8_t *)malloc((size_t)N * nblk * ORC_Q8_0_BLOCK_BYTES);
    if (!xq) return 3;
    uint8_t *wq = NULL;
    const void *wblocks = W;
    if (wtype == 2) {
        wq = (uint8_t *)malloc((size_t)M * nblk * ORC_Q8_0_BLOCK_BYTES);
        if (!wq) { free(xq); return 3; }
        orc_unrepack_q8_0(W, (int64_t)M * nblk, wq);
        wblocks = wq;
    }
    const int nt = pick_threads(nthreads);
    (void)nt;
#pragma omp parallel for schedule(static) num_threads(nt)
    for (int n = 0; n < N; ++n)
        orc_quantize_q8_0(X + (int64_t)n * K, xq + (int64_t)n * nblk * ORC_Q8_0_BLOCK_BYTES, K);
    const int rc = orc_mul_mat_q8q8(wblocks, xq, C, M, N, K, c_trans, fma, nthreads);
    free(xq);
    free(wq);
    return rc;
}

/* include/ppml/QuantBlocks.h:81-111 (host) and src/cuda/QuantKernels.cu:29-62 (device): the
 * activation quantizer of the reference's CUDA path.  Records are {half d, half s, int8 qs[32]}.
 * vmax is the first element (lowest index) that reaches the largest magnitude (strict `>` scan);
 * d = vmax / -128 keeps its sign; an all-zero block stores +0; quants clamp to [-128, 127];
 * s = half(d * float(sum of quants)) with the binary32 d. */
int orc_quantize_q8_1(const float *src, void *dst_blocks, int64_t n) {
    if (!src || !dst_blocks || n < 0 || n % ORC_QK8_0) return 1;
    uint8_t *out = (uint8_t *)dst_blocks;
    for (int64_t b = 0; b < n / ORC_QK8_0; ++b) {
        const float *x = src + b * ORC_QK8_0;
        float amax = 0.0f, vmax = 0.0f;
        for (int i = 0; i < ORC_QK8_0; ++i) {
            const float v = x[i];
            if (fabsf(v) > amax) { amax = fabsf(v); vmax = v; }
        }
        const float d = (amax == 0.0f) ? 0.0f : vmax / -128.0f;
        const float inv = (d == 0.0f) ? 0.0f : 1.0f / d;
        int32_t qsum = 0;
        uint8_t *blk = out + b * 36;
        for (int i = 0; i < ORC_QK8_0; ++i) {
            float q = roundf(x[i] * inv);
            q = q > 127.0f ? 127.0f : (q < -128.0f ? -128.0f : q);
            const int8_t qi = (int8_t)q;
            blk[4 + i] = (uint8_t)qi;
            qsum += qi;
        }
        const uint16_t dh = orc_fp32_to_fp16(d), sh = orc_fp32_to_fp16(d * (float)qsum);
        memcpy(blk, &dh, 2);
        memcpy(blk + 2, &sh, 2);
    }
    return 0;
}

/* The numbers mul_mat_q8_cuda produces (src/cuda/MulMatQ8Kernel.cu:483-527): activations quantized
 * with the Q8_1 rule above, each block settled with the halves d_w and d_a exactly like the Q8_0
 * path (120-142); s is not read.  act: 0 = Q8_0 activations (orc_mul_mat_q8), 1 = Q8_1. */
int orc_mul_mat_q8_act(const void *W, const float *X, float *C, int M, int N, int K,
                       int wtype, int c_trans, int fma, int act, int nthreads) {
    if (act == 0) return orc_mul_mat_q8(W, X, C, M, N, K, wtype, c_trans, fma, nthreads);
    if (act != 1) return 1;
    if (!W || !X || !C || M <= 0 || N <= 0 || K <= 0) return 1;
    if (K % ORC_QK8_0) return 2;
    if (wtype != 0 && wtype != 2) return 5;
    const int64_t nblk = K / ORC_QK8_0;
    uint8_t *x1 = (uint8_t *)malloc((size_t)N * nblk * 36);
    uint8_t *xq = (uint8_t *)malloc((size_t)N * nblk * ORC_Q8_0_BLOCK_BYTES);
    uint8_t *wq = NULL;
    if (!x1 || !xq) { free(x1); free(xq); return 3; }
    const void *wblocks = W;
    if (wtype == 2) {
        wq = (uint8_t *)malloc((size_t)M * nblk * ORC_Q8_0_BLOCK_BYTES);
        if (!wq) { free(x1); free(xq); return 3; }
        orc_unrepack_q8_0(W, (int64_t)M * nblk, wq);
        wblocks = wq;
    }
    orc_quantize_q8_1(X, x1, (int64_t)N * K);
    for (int64_t b = 0; b < (int64_t)N * nblk; ++b) {            /* {d, s, qs} -> {d, qs} */
        memcpy(xq + b * ORC_Q8_0_BLOCK_BYTES, x1 + b * 36, 2);
        memcpy(xq + b * ORC_Q8_0_BLOCK_BYTES + 2, x1 + b * 36 + 4, 32);
    }
    const int rc = orc_mul_mat_q8q8(wblocks, xq, C, M, N, K, c_trans, fma, nthreads);
    free(x1);
    free(xq);
    free(wq);
    return rc;
}

/* ------------------------------------------------------------------ f32 */
/* src/backend/CPUKernels.cpp:763-771: rows handed out one at a time, bias enters the
 * accumulator first, k ascending, separate multiply and add. */
void orc_mul_mat_f32(const float *a, const float *b, float *d, int M, int K, int N,
                     const float *bias, int nthreads) {
    const int nt = pick_threads(nthreads);
    (void)nt;
#pragma omp parallel for schedule(dynamic, 1) num_threads(nt)
    for (int i = 0; i < M; ++i) {
        for (int j = 0; j < N; ++j) {
            float sum = bias ? bias[j] : 0.0f;
            for (int k = 0; k < K; ++k) sum += a[(int64_t)i * K + k] * b[(int64_t)j * K + k];
            d[j + (int64_t)i * N] = sum;
        }
    }
}

/* src/backend/CPUKernels.cpp:392-396 (dot_half_row_soft) and 646-672: A and B hold halves, each
 * product is formed in binary32 (exact: two 11-bit significands), summed k ascending, and the bias
 * is added to the finished dot product.  (The reference's F16C variant keeps 8 partial sums; this
 * restates the portable one.) */
void orc_mul_mat_f16(const uint16_t *a, const uint16_t *b, float *d, int M, int K, int N,
                     const float *bias, int nthreads) {
    const int nt = pick_threads(nthreads);
    (void)nt;
#pragma omp parallel for schedule(dynamic, 1) num_threads(nt)
    for (int i = 0; i < M; ++i) {
        for (int j = 0; j < N; ++j) {
            float acc = 0.0f;
            for (int k = 0; k < K; ++k)
                acc += orc_fp16_to_fp32(a[(int64_t)i * K + k]) * orc_fp16_to_fp32(b[(int64_t)j * K + k]);
            d[j + (int64_t)i * N] = bias ? (acc + bias[j]) : acc;
        }
    }
}

/* src/backend/CPUKernels.cpp:787-887: dst zeroed, then for each dst row (i1,i2,i3)
 * d_row[i0] += s0[i0,k,i02,i03] * s1[i1,k,i2,i3], k ascending (the reference's K-blocking of
 * 32 and row-blocking of 16 leave the per-element order unchanged); src0 planes broadcast
 * with i02 = i2 / (ne2/ne02), i03 = i3 / (ne3/ne03). */
void orc_out_prod(const float *s0, const float *s1, float *dst,
                  int64_t ne00, int64_t ne01, int64_t ne02, int64_t ne03,
                  int64_t ne10, int64_t ne11, int64_t ne12, int64_t ne13,
                  int64_t ne0, int64_t ne1, int64_t ne2, int64_t ne3, int nthreads) {
    (void)ne13;
    const int64_t nr = ne1 * ne2 * ne3;
    const int64_t dps2 = ne2 / ne02;
    const int64_t dps3 = ne3 / ne03;
    const int nt = pick_threads(nthreads);
    (void)nt;
#pragma omp parallel for schedule(static) num_threads(nt)
    for (int64_t ir = 0; ir < nr; ++ir) {
        const int64_t i3 = ir / (ne2 * ne1);
        const int64_t i2 = (ir - i3 * ne2 * ne1) / ne1;
        const int64_t i1 = ir - i3 * ne2 * ne1 - i2 * ne1;
        const int64_t i02 = i2 / dps2;
        const int64_t i03 = i3 / dps3;
        float *d_row = dst + (i1 * ne0 + i2 * ne0 * ne1 + i3 * ne0 * ne1 * ne2);
        for (int64_t i0 = 0; i0 < ne0; ++i0) d_row[i0] = 0.0f;
        for (int64_t k = 0; k < ne01; ++k) {
            const float *a = s0 + (k * ne00 + i02 * ne00 * ne01 + i03 * ne00 * ne01 * ne02);
            const float bv = s1[i1 + k * ne10 + i2 * ne10 * ne11 + i3 * ne10 * ne11 * ne12];
            for (int64_t i0 = 0; i0 < ne00; ++i0) d_row[i0] += a[i0] * bv;
        }
    }
}

/* src/backend/CPUKernels.cpp:982-1032: flat output index decoded b -> j -> i -> d2 -> d1,
 * inputs indexed ((d*L + i)*N + n)*B + b, sum over n ascending, 1/N applied after the sum. */
void orc_outer_prod_mean(const float *left, const float *right, float *dst,
                         int64_t D, int64_t L, int64_t N, int64_t B, int nthreads) {
    const float inv_N = 1.0f / (float)N;
    const int64_t total = D * D * L * L * B;
    const int nt = pick_threads(nthreads);
    (void)nt;
#pragma omp parallel for schedule(static) num_threads(nt)
    for (int64_t idx = 0; idx < total; ++idx) {
        int64_t t = idx;
        const int64_t b = t % B; t /= B;
        const int64_t j = t % L; t /= L;
        const int64_t i = t % L; t /= L;
        const int64_t d2 = t % D; t /= D;
        const int64_t d1 = t;
        float sum = 0.0f;
        for (int64_t n = 0; n < N; ++n)
            sum += left[((d1 * L + i) * N + n) * B + b] * right[((d2 * L + j) * N + n) * B + b];
        dst[idx] = sum * inv_N;
    }
}

/* src/ops/MathUtils.cpp:387-437: left/right (B,N,L,D) row-major -> dst (B,L,L,D*D). */
void orc_outer_product_mean_value(const float *left, const float *right, float *dst,
                                  int64_t B, int64_t N, int64_t L, int64_t D, int nthreads) {
    const float inv_N = 1.0f / (float)N;
    const int64_t D2 = D * D;
    const int nt = pick_threads(nthreads);
    (void)nt;
#pragma omp parallel for schedule(static) collapse(2) num_threads(nt)
    for (int64_t b = 0; b < B; ++b)
        for (int64_t i = 0; i < L; ++i)
            for (int64_t j = 0; j < L; ++j)
                for (int64_t d1 = 0; d1 < D; ++d1)
                    for (int64_t d2 = 0; d2 < D; ++d2) {
                        float sum = 0.0f;
                        for (int64_t n = 0; n < N; ++n)
                            sum += left[((b * N + n) * L + i) * D + d1] *
                                   right[((b * N + n) * L + j) * D + d2];
                        dst[((b * L + i) * L + j) * D2 + (d1 * D + d2)] = sum * inv_N;
                    }
}

/* src/modules/Attention.cpp:58-79: Q,K value layout (NQ,H,D,L); scores (NQ,H,Lq,Lk),
 * scaled by 1/sqrt(D) after the sum. */
void orc_attention_scores(const float *Q, const float *K, float *scores,
                          int64_t NQ, int64_t H, int64_t D, int64_t Lq, int64_t Lk, int nthreads) {
    const float inv_scale = 1.0f / sqrtf((float)D);
    const int nt = pick_threads(nthreads);
    (void)nt;
#pragma omp parallel for schedule(static) collapse(2) num_threads(nt)
    for (int64_t b = 0; b < NQ; ++b)
        for (int64_t h = 0; h < H; ++h)
            for (int64_t i = 0; i < Lq; ++i)
                for (int64_t j = 0; j < Lk; ++j) {
                    float s = 0.0f;
                    const float *qp = Q + ((b * H + h) * D) * Lq + i;
                    const float *kp = K + ((b * H + h) * D) * Lk + j;
                    for (int64_t d = 0; d < D; ++d) s += qp[d * Lq] * kp[d * Lk];
                    scores[((b * H + h) * Lq + i) * Lk + j] = s * inv_scale;
                }
}

/* src/backend/CPUKernels.cpp:2091-2148 (kernel_repeat_back).  nd_src / nd_dst are the tensors' ranks, sd_in /
 * dd_in their sizes (dims[0] innermost; entries past the rank ignored).  Dimension d of dst meets dimension
 * d of src (2108); the number of copies per dimension is the integer quotient of the sizes (2117-2122); every
 * destination element is the sum of its copies added one at a time, k0 outermost, k3 innermost (2139-2151). */
void orc_repeat_back(const float *src, float *dst, int nd_src, const int64_t sd_in[4], int nd_dst, const int64_t dd_in[4]) {
    const int off = (nd_src >= nd_dst) ? 0 : (nd_src - nd_dst);
    int64_t dd[4] = {1, 1, 1, 1}, sd[4] = {1, 1, 1, 1}, rd[4] = {1, 1, 1, 1};
    for (int d = 0; d < nd_dst && d < 4; ++d) dd[d] = dd_in[d];
    for (int d = 0; d < nd_src && d < 4; ++d) sd[d] = sd_in[d];
    for (int d = 0; d < 4; ++d) {
        const int s_idx = d + off;
        const int64_t sdim = (s_idx >= 0 && s_idx < 4) ? sd[s_idx] : 1;
        rd[d] = dd[d] > 0 ? sdim / dd[d] : 1;
    }
    const int64_t total = dd[0] * dd[1] * dd[2] * dd[3];
    for (int64_t idx = 0; idx < total; ++idx) {
        int64_t t = idx;
        const int64_t j0 = t % dd[0]; t /= dd[0];
        const int64_t j1 = t % dd[1]; t /= dd[1];
        const int64_t j2 = t % dd[2]; t /= dd[2];
        const int64_t j3 = t;
        float sum = 0.0f;
        for (int64_t k0 = 0; k0 < rd[0]; ++k0)
            for (int64_t k1 = 0; k1 < rd[1]; ++k1)
                for (int64_t k2 = 0; k2 < rd[2]; ++k2)
                    for (int64_t k3 = 0; k3 < rd[3]; ++k3) {
                        const int64_t s0 = j0 + k0 * dd[0], s1 = j1 + k1 * dd[1], s2 = j2 + k2 * dd[2], s3 = j3 + k3 * dd[3];
                        sum += src[((s3 * sd[2] + s2) * sd[1] + s1) * sd[0] + s0];
                    }
        dst[idx] = sum;
    }
}

/* src/backend/CPUKernels.cpp:1737-1754 (kernel_scale): dst[i] = src[i] * s, s from op_params[0]. */
void orc_scale(const float *src, float *dst, int64_t n, float s, int nthreads) {
    const int nt = pick_threads(nthreads);
    (void)nt;
#pragma omp parallel for schedule(static) num_threads(nt)
    for (int64_t i = 0; i < n; ++i) dst[i] = src[i] * s;
}

/* src/backend/CPUKernels.cpp:2649-2657 (compute_forward_relu): d = (s > 0) ? s : 0 -- NaN and -0 give +0. */
void orc_relu(const float *src, float *dst, int64_t n, int nthreads) {
    const int nt = pick_threads(nthreads);
    (void)nt;
#pragma omp parallel for schedule(static) num_threads(nt)
    for (int64_t i = 0; i < n; ++i) dst[i] = (src[i] > 0.0f) ? src[i] : 0.0f;
}

/* src/backend/CPUKernels.cpp:446-596 (kernel_elemwise): d[i] = a[a_full ? i : i % an] op b[b_full ? i : i % bn]
 * (549-592); eop 0 add, 1 sub, 2 mul, 3 div as the CUDA wrapper numbers them (src/backend/CUDAKernels.cpp:678-712).
 * The AVX2 branch of OP_ADD (542-548) adds the same pairs.  returns 0 ok, 1 bad arguments. */
int orc_bcast_elemwise(const float *a, const float *b, float *d, int64_t n, int64_t an, int64_t bn, int eop, int nthreads) {
    if (!a || !b || !d || n < 0 || an <= 0 || bn <= 0 || eop < 0 || eop > 3) return 1;
    const int a_full = an == n, b_full = bn == n;
    const int nt = pick_threads(nthreads);
    (void)nt;
#pragma omp parallel for schedule(static) num_threads(nt)
    for (int64_t i = 0; i < n; ++i) {
        const float x = a[a_full ? i : i % an], y = b[b_full ? i : i % bn];
        d[i] = eop == 0 ? x + y : eop == 1 ? x - y : eop == 2 ? x * y : x / y;
    }
    return 0;
}

/* src/backend/CPUKernels.cpp:1446-1467 (kernel_softmax): rows of D = dims[0] values; maximum from the first
 * element moved by `>` (1459-1460), sum of expf(x - mx) d ascending (1461-1462), inv = 1 / (sum + 1e-9f) (1463),
 * expf recomputed for the output (1464). */
void orc_softmax(const float *src, float *dst, int64_t rows, int64_t D, int nthreads) {
    const int nt = pick_threads(nthreads);
    (void)nt;
#pragma omp parallel for schedule(static) num_threads(nt)
    for (int64_t r = 0; r < rows; ++r) {
        const float *sr = src + r * D;
        float *dr = dst + r * D;
        float mx = sr[0];
        for (int64_t d = 1; d < D; ++d) if (sr[d] > mx) mx = sr[d];
        float sum = 0;
        for (int64_t d = 0; d < D; ++d) sum += expf(sr[d] - mx);
        const float inv = 1.0f / (sum + 1e-9f);
        for (int64_t d = 0; d < D; ++d) dr[d] = expf(sr[d] - mx) * inv;
    }
}
