// True-fp32 MFMA contractions for gfx950: dense GEMM with bias (mul_mat), batched transposed
// GEMM with plane broadcast (out_prod, attention logits) and outer-product-mean in both of the
// reference's layouts.  One kernel, three operand-access modes.
//
// Reference behaviour restated here (paths relative to the reference tree):
//   mul_mat          src/backend/CPUKernels.cpp:763-771   (bias first, k ascending)
//   out_prod         src/backend/CPUKernels.cpp:787-887
//   outer_prod_mean  src/backend/CPUKernels.cpp:982-1032, src/ops/MathUtils.cpp:387-437
//
// Reduction order: every output is accumulated in fp32 by v_mfma_f32_32x32x2_f32, k ascending in
// steps of 2 (the instruction adds a[k]*b[k] + a[k+1]*b[k+1] to the accumulator), starting from
// bias[n] (or 0); alpha multiplies the finished sum.
#include "common.hpp"

namespace ppmlhip {
namespace {

constexpr int BM = 128, BN = 128, BK = 16;
constexpr int LDS_LD = BM + 4;        // row pitch of the k-major LDS tiles (floats)

enum LoadMode { LOAD_K_CONTIG = 0, LOAD_ROW_CONTIG = 1, LOAD_STRIDED = 2, LOAD_K_CONTIG_F16 = 3, LOAD_SPLIT_A = 4 };

struct GemmParams {
    const float* A;       // rows m: A(m,k) = A[m*a_rs + k*a_ks]
    const float* B;       // cols n: B(n,k) = B[n*b_rs + k*b_ks]
    float* C;
    const float* bias;    // [N] or null
    int M, N, K;
    int64_t a_rs, a_ks, b_rs, b_ks;
    // planes: p = p3*np2 + p2
    int np2, np3;
    int64_t a_p2, a_p3, b_p2, b_p3, c_p2, c_p3;
    int b_div2, b_div3;   // B-side plane index = p / div (out_prod's src0 broadcast)
    float alpha;
    // C(m,n) = C[(m/c_lm)*c_mo + (m%c_lm)*c_mi + (n/c_ln)*c_no + (n%c_ln)*c_ni]
    int c_lm, c_ln;
    int64_t c_mo, c_mi, c_no, c_ni;
    int tiles_m, tiles_n;
    int stream_c;         // output larger than the last-level cache: write it with streaming stores
    int f16_in;           // A and B hold IEEE halves (k contiguous); products and sums are binary32
    int clamp;            // finite guard in the epilogue (triangle multiplication)
    // LOAD_SPLIT_A: both indices of A are compound, A(m,k) = A[(m/a_lm)*a_mo + (m%a_lm)*a_mi + (k/a_lk)*a_ko + (k%a_lk)*a_ki]
    int a_lm, a_lk;
    int64_t a_mo, a_mi, a_ko, a_ki;
};

// 16 x 128 tile of one operand -> two v4f per thread
template <int MODE>
__device__ __forceinline__ void load_tile(const float* __restrict__ base, int64_t rs, int64_t ks,
                                          int row0, int nrows, int k0, int K, int tid, v4f (&reg)[2]) {
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        v4f v = {0.f, 0.f, 0.f, 0.f};
        if (MODE == LOAD_K_CONTIG) {
            const int r = (tid >> 2) + it * 64;          // row within tile
            const int k = k0 + (tid & 3) * 4;
            const int row = row0 + r;
            if (row < nrows) {
                const float* p = base + static_cast<int64_t>(row) * rs + k;
                if (k + 3 < K) v = *reinterpret_cast<const v4f_u*>(p);
                else {
#pragma unroll
                    for (int c = 0; c < 4; ++c) if (k + c < K) v[c] = p[c];
                }
            }
        } else if (MODE == LOAD_K_CONTIG_F16) {
            // the same tile shape read from halves: 4 of them (8 bytes) per thread and pass
            const int r = (tid >> 2) + it * 64;
            const int k = k0 + (tid & 3) * 4;
            const int row = row0 + r;
            if (row < nrows) {
                const __half* p = reinterpret_cast<const __half*>(base) + static_cast<int64_t>(row) * rs + k;
                if (k + 3 < K && (reinterpret_cast<uintptr_t>(p) & 7) == 0) {
                    const uint2 raw = *reinterpret_cast<const uint2*>(p);
                    const __half2 lo = *reinterpret_cast<const __half2*>(&raw.x), hi = *reinterpret_cast<const __half2*>(&raw.y);
                    v[0] = __low2float(lo); v[1] = __high2float(lo); v[2] = __low2float(hi); v[3] = __high2float(hi);
                } else {
#pragma unroll
                    for (int c = 0; c < 4; ++c) if (k + c < K) v[c] = __half2float(p[c]);
                }
            }
        } else if (MODE == LOAD_ROW_CONTIG) {
            const int kk = (tid >> 5) + it * 8;
            const int r = (tid & 31) * 4;
            const int k = k0 + kk, row = row0 + r;
            if (k < K) {
                const float* p = base + static_cast<int64_t>(k) * ks + row;
                if (row + 3 < nrows) v = *reinterpret_cast<const v4f_u*>(p);
                else {
#pragma unroll
                    for (int c = 0; c < 4; ++c) if (row + c < nrows) v[c] = p[c];
                }
            }
        } else {
            const int r = (tid >> 2) + it * 64;
            const int k = k0 + (tid & 3) * 4;
            const int row = row0 + r;
            if (row < nrows) {
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    if (k + c < K) v[c] = base[static_cast<int64_t>(row) * rs + static_cast<int64_t>(k + c) * ks];
            }
        }
        reg[it] = v;
    }
}

// A tile of an operand whose row and contraction indices are both compound (the gradient tensor of the
// outer-product-mean backward, indexed [d1][d2][i][j]): one element at a time.
__device__ __forceinline__ void load_tile_split(const float* __restrict__ base, const GemmParams& p,
                                                int row0, int nrows, int k0, int K, int tid, v4f (&reg)[2]) {
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        v4f v = {0.f, 0.f, 0.f, 0.f};
        const int row = row0 + (tid >> 2) + it * 64;
        const int k = k0 + (tid & 3) * 4;
        if (row < nrows) {
            const int64_t roff = static_cast<int64_t>(row / p.a_lm) * p.a_mo + static_cast<int64_t>(row % p.a_lm) * p.a_mi;
#pragma unroll
            for (int c = 0; c < 4; ++c)
                if (k + c < K) v[c] = base[roff + static_cast<int64_t>((k + c) / p.a_lk) * p.a_ko + static_cast<int64_t>((k + c) % p.a_lk) * p.a_ki];
        }
        reg[it] = v;
    }
}

template <int MODE>
__device__ __forceinline__ void store_tile(float* __restrict__ lds, int tid, const v4f (&reg)[2]) {
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        if (MODE == LOAD_ROW_CONTIG) {
            const int kk = (tid >> 5) + it * 8;
            const int r = (tid & 31) * 4;
            *reinterpret_cast<v4f*>(lds + kk * LDS_LD + r) = reg[it];
        } else {
            const int r = (tid >> 2) + it * 64;
            const int kk = (tid & 3) * 4;
#pragma unroll
            for (int c = 0; c < 4; ++c) lds[(kk + c) * LDS_LD + r] = reg[it][c];
        }
    }
}

// CLAMP: the finite guard of the triangle multiplication (src/backend/CPUKernels.cpp:957-962): NaN -> 0,
// values beyond +-1e4 -> +-1e4.  A compile-time property: a run-time test in this store loop costs the
// other contractions a quarter of their speed.
template <int MODE, bool SPLIT_C, bool STREAM_C, bool CLAMP = false>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const GemmParams p) {
    __shared__ __attribute__((aligned(16))) float lds_a[BK * LDS_LD];
    __shared__ __attribute__((aligned(16))) float lds_b[BK * LDS_LD];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int j = lane & 31, hh = lane >> 5;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;

    // work-group -> (plane, tile row, tile col); bands of 8 tile rows keep operand panels in one L2
    const int tiles = p.tiles_m * p.tiles_n;
    const int total = tiles * p.np2 * p.np3;
    const int idx = xcd_contiguous_index(blockIdx.x, total);
    const int plane = idx / tiles;
    int t = idx - plane * tiles;
    const int band_rows = 8;
    const int band = t / (band_rows * p.tiles_n);
    t -= band * band_rows * p.tiles_n;
    const int rows_here = (p.tiles_m - band * band_rows) < band_rows ? (p.tiles_m - band * band_rows) : band_rows;
    const int tm = band * band_rows + t % rows_here;
    const int tn = t / rows_here;
    const int m0 = tm * BM, n0 = tn * BN;

    const int p2 = plane % p.np2, p3 = plane / p.np2;
    const float* A = p.A + p2 * p.a_p2 + p3 * p.a_p3;
    const float* B = p.B + (p2 / p.b_div2) * p.b_p2 + (p3 / p.b_div3) * p.b_p3;
    float* C = p.C + p2 * p.c_p2 + p3 * p.c_p3;

    // halves in: the bias joins the finished sum (the CPU branch of the reference adds it last)
    constexpr bool BIAS_LAST = MODE == LOAD_K_CONTIG_F16;
    v16f acc[2][2];
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) {
        const int n = n0 + wn + tj * 32 + j;
        const float b0 = (p.bias && !BIAS_LAST && n < p.N) ? p.bias[n] : 0.0f;
#pragma unroll
        for (int ti = 0; ti < 2; ++ti)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[ti][tj][r] = b0;
    }

    v4f ra[2], rb[2];
    constexpr int MODE_B = MODE == LOAD_SPLIT_A ? LOAD_STRIDED : MODE;
    if (MODE == LOAD_SPLIT_A) load_tile_split(A, p, m0, p.M, 0, p.K, tid, ra);
    else load_tile<MODE>(A, p.a_rs, p.a_ks, m0, p.M, 0, p.K, tid, ra);
    load_tile<MODE_B>(B, p.b_rs, p.b_ks, n0, p.N, 0, p.K, tid, rb);

    for (int k0 = 0; k0 < p.K; k0 += BK) {
        store_tile<MODE>(lds_a, tid, ra);
        store_tile<MODE>(lds_b, tid, rb);
        __syncthreads();
        if (k0 + BK < p.K) {
            if (MODE == LOAD_SPLIT_A) load_tile_split(A, p, m0, p.M, k0 + BK, p.K, tid, ra);
            else load_tile<MODE>(A, p.a_rs, p.a_ks, m0, p.M, k0 + BK, p.K, tid, ra);
            load_tile<MODE_B>(B, p.b_rs, p.b_ks, n0, p.N, k0 + BK, p.K, tid, rb);
        }
#pragma unroll
        for (int kk = 0; kk < BK; kk += 2) {
            const float a0 = lds_a[(kk + hh) * LDS_LD + wm + j];
            const float a1 = lds_a[(kk + hh) * LDS_LD + wm + 32 + j];
            const float b0 = lds_b[(kk + hh) * LDS_LD + wn + j];
            const float b1 = lds_b[(kk + hh) * LDS_LD + wn + 32 + j];
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
        }
        __syncthreads();
    }

    const bool scale = p.alpha != 1.0f;
#pragma unroll
    for (int ti = 0; ti < 2; ++ti)
#pragma unroll
        for (int tj = 0; tj < 2; ++tj) {
            const int n = n0 + wn + tj * 32 + j;
            if (n >= p.N) continue;
            const float tail_bias = (BIAS_LAST && p.bias) ? p.bias[n] : 0.0f;
            int64_t coff;
            if (SPLIT_C) coff = static_cast<int64_t>(n / p.c_ln) * p.c_no + static_cast<int64_t>(n % p.c_ln) * p.c_ni;
            else         coff = static_cast<int64_t>(n) * p.c_ni;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm + ti * 32 + mfma32_row(r, lane);
                if (m >= p.M) continue;
                int64_t roff;
                if (SPLIT_C) roff = static_cast<int64_t>(m / p.c_lm) * p.c_mo + static_cast<int64_t>(m % p.c_lm) * p.c_mi;
                else         roff = static_cast<int64_t>(m) * p.c_mi;
                float v = acc[ti][tj][r];
                if (scale) v *= p.alpha;
                if (BIAS_LAST) v += tail_bias;
                if (CLAMP) v = (v != v) ? 0.0f : (v > 1e4f ? 1e4f : (v < -1e4f ? -1e4f : v));
                if (STREAM_C) __builtin_nontemporal_store(v, &C[roff + coff]);
                else C[roff + coff] = v;
            }
        }
}

int launch_gemm(GemmParams p, hipStream_t stream, const char* what) {
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    // An output that fits the 256 MB last-level cache is likely read next by the consumer node (the
    // logits by their softmax); a larger one only evicts useful lines on its way to HBM.  Measured:
    // streaming stores 72 -> 63 us on the 216 MB MSA logits, 14 -> 16 us on the 17 MB pair logits.
    p.stream_c = static_cast<int64_t>(p.M) * p.N * p.np2 * p.np3 * 4 >= (128LL << 20);
    const int64_t total = static_cast<int64_t>(p.tiles_m) * p.tiles_n * p.np2 * p.np3;
    if (total <= 0 || total > 0x7fffffffLL) { set_error("%s: grid of %lld work-groups is out of range", what, (long long)total); return RC_BAD_ARGS; }
    const dim3 grid(static_cast<unsigned>(total)), block(256);
    const bool split = !(p.c_lm >= p.M && p.c_ln >= p.N);
    int mode = LOAD_STRIDED;
    if (p.a_ks == 1 && p.b_ks == 1) mode = LOAD_K_CONTIG;
    else if (p.a_rs == 1 && p.b_rs == 1) mode = LOAD_ROW_CONTIG;
#define PPML_LAUNCH(MODE, SPLIT)                                                                      \
    do {                                                                                              \
        if (p.stream_c) hipLaunchKernelGGL((gemm_f32_kernel<MODE, SPLIT, true>), grid, block, 0, stream, p);  \
        else hipLaunchKernelGGL((gemm_f32_kernel<MODE, SPLIT, false>), grid, block, 0, stream, p);    \
    } while (0)
    if (p.a_lm > 0) {
        if (split || p.f16_in || p.clamp) { set_error("%s: no split-operand instance for this addressing", what); return RC_BAD_ARGS; }
        PPML_LAUNCH(LOAD_SPLIT_A, false);
    }
    else if (p.clamp) {
        if (split || p.stream_c || p.f16_in) { set_error("%s: no clamped instance for this addressing", what); return RC_BAD_ARGS; }
        if (mode == LOAD_K_CONTIG) hipLaunchKernelGGL((gemm_f32_kernel<LOAD_K_CONTIG, false, false, true>), grid, block, 0, stream, p);
        else if (mode == LOAD_ROW_CONTIG) hipLaunchKernelGGL((gemm_f32_kernel<LOAD_ROW_CONTIG, false, false, true>), grid, block, 0, stream, p);
        else hipLaunchKernelGGL((gemm_f32_kernel<LOAD_STRIDED, false, false, true>), grid, block, 0, stream, p);
    }
    else if (p.f16_in)                { PPML_LAUNCH(LOAD_K_CONTIG_F16, false); }
    else if (mode == LOAD_K_CONTIG)   { if (split) PPML_LAUNCH(LOAD_K_CONTIG, true);   else PPML_LAUNCH(LOAD_K_CONTIG, false); }
    else if (mode == LOAD_ROW_CONTIG) { if (split) PPML_LAUNCH(LOAD_ROW_CONTIG, true); else PPML_LAUNCH(LOAD_ROW_CONTIG, false); }
    else                              { if (split) PPML_LAUNCH(LOAD_STRIDED, true);    else PPML_LAUNCH(LOAD_STRIDED, false); }
#undef PPML_LAUNCH
    return check_launch(what);
}

GemmParams plain_params() {
    GemmParams p{};
    p.np2 = p.np3 = 1;
    p.b_div2 = p.b_div3 = 1;
    p.alpha = 1.0f;
    p.c_lm = p.c_ln = 0x7fffffff;
    return p;
}

}  // namespace
}  // namespace ppmlhip

using namespace ppmlhip;

extern "C" int mul_mat_hip(const float* A, const float* B, float* C, int M, int K, int N,
                           const float* bias, ppml_hip_stream_t stream) {
    if (!A || !B || !C || M <= 0 || K <= 0 || N <= 0) { set_error("mul_mat_hip: bad arguments (M=%d K=%d N=%d)", M, K, N); return RC_BAD_ARGS; }
    stats_record(M, K, N);
    GemmParams p = plain_params();
    p.A = A; p.B = B; p.C = C; p.bias = bias;
    p.M = M; p.N = N; p.K = K;
    p.a_rs = K; p.a_ks = 1; p.b_rs = K; p.b_ks = 1;
    p.c_mi = N; p.c_ni = 1;
    return launch_gemm(p, static_cast<hipStream_t>(stream), "mul_mat_hip");
}

extern "C" int mul_mat_f16_hip(const void* A16, const void* B16, float* C, int M, int K, int N,
                               const float* bias, ppml_hip_stream_t stream) {
    if (!A16 || !B16 || !C || M <= 0 || K <= 0 || N <= 0) { set_error("mul_mat_f16_hip: bad arguments (M=%d K=%d N=%d)", M, K, N); return RC_BAD_ARGS; }
    stats_record(M, K, N);
    GemmParams p = plain_params();
    p.A = static_cast<const float*>(A16); p.B = static_cast<const float*>(B16); p.C = C; p.bias = bias;
    p.M = M; p.N = N; p.K = K;
    p.a_rs = K; p.a_ks = 1; p.b_rs = K; p.b_ks = 1;      // strides in elements (halves)
    p.c_mi = N; p.c_ni = 1;
    p.f16_in = 1;
    return launch_gemm(p, static_cast<hipStream_t>(stream), "mul_mat_f16_hip");
}

extern "C" int mul_mat_tn_hip(const float* A, const float* Bm, float* O, int M, int K, int Nc, float alpha,
                              ppml_hip_stream_t stream) {
    if (!A || !Bm || !O || M <= 0 || K <= 0 || Nc <= 0) { set_error("mul_mat_tn_hip: bad arguments"); return RC_BAD_ARGS; }
    stats_record(M, K, Nc);
    GemmParams p = plain_params();
    p.A = A; p.B = Bm; p.C = O;
    p.M = M; p.N = Nc; p.K = K;
    p.a_rs = 1; p.a_ks = M; p.b_rs = 1; p.b_ks = Nc;
    p.c_mi = Nc; p.c_ni = 1;
    p.alpha = alpha;
    return launch_gemm(p, static_cast<hipStream_t>(stream), "mul_mat_tn_hip");
}

extern "C" int out_prod_scaled_hip(const float* src0, const float* src1, float* dst,
                                   int64_t ne00, int64_t ne01, int64_t ne02, int64_t ne03,
                                   int64_t ne10, int64_t ne11, int64_t ne12, int64_t ne13,
                                   int64_t ne0, int64_t ne1, int64_t ne2, int64_t ne3,
                                   float scale, ppml_hip_stream_t stream) {
    if (!src0 || !src1 || !dst) { set_error("out_prod_hip: null pointer"); return RC_BAD_ARGS; }
    const bool pos = ne00 > 0 && ne01 > 0 && ne02 > 0 && ne03 > 0 && ne10 > 0 && ne11 > 0 && ne12 > 0 && ne13 > 0;
    // shape contract of the graph builder (src/core/ComputeGraphHelper.cpp:318-345) and the
    // broadcast rule of the CPU kernel (src/backend/CPUKernels.cpp:836-837)
    if (!pos || ne01 != ne11 || ne0 != ne00 || ne1 != ne10 || ne2 != ne12 || ne3 != ne13 ||
        ne2 % ne02 != 0 || ne3 % ne03 != 0 || ne0 > 0x7fffffff || ne1 > 0x7fffffff || ne01 > 0x7fffffff) {
        set_error("out_prod_hip: shape mismatch src0[%lld,%lld,%lld,%lld] src1[%lld,%lld,%lld,%lld] dst[%lld,%lld,%lld,%lld]",
                  (long long)ne00, (long long)ne01, (long long)ne02, (long long)ne03,
                  (long long)ne10, (long long)ne11, (long long)ne12, (long long)ne13,
                  (long long)ne0, (long long)ne1, (long long)ne2, (long long)ne3);
        return RC_BAD_ARGS;
    }
    stats_record(ne1, ne01, ne0);
    GemmParams p = plain_params();
    p.A = src1; p.B = src0; p.C = dst;                 // rows = i1 (src1), cols = i0 (src0)
    p.M = static_cast<int>(ne1); p.N = static_cast<int>(ne0); p.K = static_cast<int>(ne01);
    p.a_rs = 1; p.a_ks = ne10; p.b_rs = 1; p.b_ks = ne00;
    p.np2 = static_cast<int>(ne2); p.np3 = static_cast<int>(ne3);
    p.a_p2 = ne10 * ne11; p.a_p3 = ne10 * ne11 * ne12;
    p.b_p2 = ne00 * ne01; p.b_p3 = ne00 * ne01 * ne02;
    p.c_p2 = ne0 * ne1;   p.c_p3 = ne0 * ne1 * ne2;
    p.b_div2 = static_cast<int>(ne2 / ne02); p.b_div3 = static_cast<int>(ne3 / ne03);
    p.c_mi = ne0; p.c_ni = 1;
    p.alpha = scale;
    return launch_gemm(p, static_cast<hipStream_t>(stream), "out_prod_hip");
}

extern "C" int out_prod_hip(const float* src0, const float* src1, float* dst,
                            int64_t ne00, int64_t ne01, int64_t ne02, int64_t ne03,
                            int64_t ne10, int64_t ne11, int64_t ne12, int64_t ne13,
                            int64_t ne0, int64_t ne1, int64_t ne2, int64_t ne3,
                            ppml_hip_stream_t stream) {
    return out_prod_scaled_hip(src0, src1, dst, ne00, ne01, ne02, ne03, ne10, ne11, ne12, ne13,
                               ne0, ne1, ne2, ne3, 1.0f, stream);
}

extern "C" int outer_prod_mean_hip(const float* left, const float* right, float* dst,
                                   int64_t D, int64_t L, int64_t N, int64_t B, float inv_N,
                                   ppml_hip_stream_t stream) {
    if (!left || !right || !dst || D <= 0 || L <= 0 || N <= 0 || B <= 0 || D * L > 0x7fffffff || N > 0x7fffffff) {
        set_error("outer_prod_mean_hip: bad arguments"); return RC_BAD_ARGS;
    }
    stats_record(D * L, N, D * L);
    GemmParams p = plain_params();
    p.A = left; p.B = right; p.C = dst;               // rows = (d1,i), cols = (d2,j), k = n
    p.M = p.N = static_cast<int>(D * L); p.K = static_cast<int>(N);
    p.a_rs = N * B; p.a_ks = B; p.b_rs = N * B; p.b_ks = B;
    p.np2 = static_cast<int>(B);                       // batch b is the innermost index of every tensor
    p.a_p2 = 1; p.b_p2 = 1; p.c_p2 = 1;
    p.alpha = inv_N;
    p.c_lm = p.c_ln = static_cast<int>(L);
    p.c_mo = D * L * L * B; p.c_mi = L * B; p.c_no = L * L * B; p.c_ni = B;
    return launch_gemm(p, static_cast<hipStream_t>(stream), "outer_prod_mean_hip");
}

extern "C" int outer_product_mean_value_hip(const float* left, const float* right, float* dst,
                                            int64_t B, int64_t N, int64_t L, int64_t D,
                                            ppml_hip_stream_t stream) {
    if (!left || !right || !dst || D <= 0 || L <= 0 || N <= 0 || B <= 0 || D * L > 0x7fffffff || N > 0x7fffffff) {
        set_error("outer_product_mean_value_hip: bad arguments"); return RC_BAD_ARGS;
    }
    stats_record(D * L, N, D * L);
    GemmParams p = plain_params();
    p.A = left; p.B = right; p.C = dst;               // rows = (i,d1), cols = (j,d2), k = n
    p.M = p.N = static_cast<int>(L * D); p.K = static_cast<int>(N);
    p.a_rs = 1; p.a_ks = L * D; p.b_rs = 1; p.b_ks = L * D;
    p.np2 = static_cast<int>(B);
    p.a_p2 = N * L * D; p.b_p2 = N * L * D; p.c_p2 = L * L * D * D;
    p.alpha = 1.0f / static_cast<float>(N);
    p.c_lm = p.c_ln = static_cast<int>(D);
    p.c_mo = L * D * D; p.c_mi = D; p.c_no = D * D; p.c_ni = 1;
    return launch_gemm(p, static_cast<hipStream_t>(stream), "outer_product_mean_value_hip");
}

extern "C" int tri_mul_hip(const float* left, const float* right, float* dst,
                           int64_t D, int64_t I, int64_t J, int64_t K, int64_t B, float inv_L, int outgoing,
                           ppml_hip_stream_t stream) {
    if (!left || !right || !dst || D <= 0 || I <= 0 || J <= 0 || K <= 0 || B <= 0 ||
        I > 0x7fffffff || J > 0x7fffffff || K > 0x7fffffff || D > 0x7fffffff || B > 0x7fffffff) {
        set_error("tri_mul_hip: bad arguments"); return RC_BAD_ARGS;
    }
    stats_record(I, K, J);
    GemmParams p = plain_params();
    p.A = left; p.B = right; p.C = dst;                // rows = i, cols = j, planes = (d, b)
    p.M = static_cast<int>(I); p.N = static_cast<int>(J); p.K = static_cast<int>(K);
    if (outgoing) {                                    // left[((d*I+i)*K+k)*B+b], right[((d*J+j)*K+k)*B+b]
        p.a_rs = K * B; p.a_ks = B; p.b_rs = K * B; p.b_ks = B;
    } else {                                           // left[((d*K+k)*I+i)*B+b], right[((d*K+k)*J+j)*B+b]
        p.a_rs = B; p.a_ks = I * B; p.b_rs = B; p.b_ks = J * B;
    }
    p.np2 = static_cast<int>(B); p.np3 = static_cast<int>(D);
    p.a_p2 = 1; p.b_p2 = 1; p.c_p2 = 1;                // batch b is the innermost index of every tensor
    p.a_p3 = I * K * B; p.b_p3 = J * K * B; p.c_p3 = I * J * B;
    p.c_mi = J * B; p.c_ni = B;                        // dst[((d*I+i)*J+j)*B+b]
    p.alpha = inv_L;
    p.clamp = 1;
    return launch_gemm(p, static_cast<hipStream_t>(stream), "tri_mul_hip");
}

extern "C" int tri_mul_back_hip(const float* grad, const float* left, const float* right, float* gleft, float* gright,
                                int64_t D, int64_t I, int64_t J, int64_t K, int64_t B, float inv_L, int outgoing,
                                ppml_hip_stream_t stream) {
    if (!grad || !left || !right || (!gleft && !gright) || D <= 0 || I <= 0 || J <= 0 || K <= 0 || B <= 0 ||
        I > 0x7fffffff || J > 0x7fffffff || K > 0x7fffffff || D > 0x7fffffff || B > 0x7fffffff) {
        set_error("tri_mul_back_hip: bad arguments"); return RC_BAD_ARGS;
    }
    // Per (d, b) plane, with grad[i][j] = grad[((d*I+i)*J+j)*B+b]:
    //   outgoing  gleft[i][k]  = sum_j grad[i][j] * right[j][k]     gright[j][k] = sum_i grad[i][j] * left[i][k]
    //   incoming  gleft[k][i]  = sum_j grad[i][j] * right[k][j]     gright[k][j] = sum_i grad[i][j] * left[k][i]
    // Every one is a contraction with one stride per operand index, i.e. a launch of the strided kernel.
    const auto launch = [&](const float* a, int64_t a_rs, int64_t a_ks, const float* b, int64_t b_rs, int64_t b_ks,
                            float* c, int64_t c_mi, int64_t c_ni, int64_t M, int64_t N, int64_t Kc,
                            int64_t a_p3, int64_t b_p3, int64_t c_p3) {
        stats_record(M, Kc, N);
        GemmParams p = plain_params();
        p.A = a; p.B = b; p.C = c;
        p.M = static_cast<int>(M); p.N = static_cast<int>(N); p.K = static_cast<int>(Kc);
        p.a_rs = a_rs * B; p.a_ks = a_ks * B; p.b_rs = b_rs * B; p.b_ks = b_ks * B;
        p.c_mi = c_mi * B; p.c_ni = c_ni * B;
        p.np2 = static_cast<int>(B); p.np3 = static_cast<int>(D);
        p.a_p2 = 1; p.b_p2 = 1; p.c_p2 = 1;
        p.a_p3 = a_p3 * B; p.b_p3 = b_p3 * B; p.c_p3 = c_p3 * B;
        p.alpha = inv_L;
        return launch_gemm(p, static_cast<hipStream_t>(stream), "tri_mul_back_hip");
    };
    int rc = RC_OK;
    if (outgoing) {
        if (gleft)  rc = launch(grad, J, 1, right, 1, K, gleft, K, 1, I, K, J, I * J, J * K, I * K);
        if (rc == RC_OK && gright) rc = launch(grad, 1, J, left, 1, K, gright, K, 1, J, K, I, I * J, I * K, J * K);
    } else {
        if (gleft)  rc = launch(grad, J, 1, right, J, 1, gleft, 1, I, I, K, J, I * J, K * J, K * I);
        if (rc == RC_OK && gright) rc = launch(grad, 1, J, left, I, 1, gright, 1, J, J, K, I, I * J, K * I, K * J);
    }
    return rc;
}

extern "C" int outer_prod_mean_back_hip(const float* grad, const float* left, const float* right, float* gleft, float* gright,
                                        int64_t D, int64_t L, int64_t N, int64_t B, float inv_N, ppml_hip_stream_t stream) {
    if (!grad || !left || !right || (!gleft && !gright) || D <= 0 || L <= 0 || N <= 0 || B <= 0 ||
        D * L > 0x7fffffff || N > 0x7fffffff || B > 0x7fffffff) {
        set_error("outer_prod_mean_back_hip: bad arguments"); return RC_BAD_ARGS;
    }
    // grad[d1][d2][i][j][b]; gleft[(d1,i)][n] = inv_N * sum_{(d2,j)} grad * right[(d2,j)][n],
    //                        gright[(d2,j)][n] = inv_N * sum_{(d1,i)} grad * left[(d1,i)][n]:
    // two contractions whose first operand has a compound row index and a compound contraction index.
    const auto launch = [&](const float* other, float* out, int64_t mo, int64_t mi, int64_t ko, int64_t ki) {
        stats_record(D * L, D * L, N);
        GemmParams p = plain_params();
        p.A = grad; p.B = other; p.C = out;
        p.M = static_cast<int>(D * L); p.N = static_cast<int>(N); p.K = static_cast<int>(D * L);
        p.a_lm = p.a_lk = static_cast<int>(L);
        p.a_mo = mo * B; p.a_mi = mi * B; p.a_ko = ko * B; p.a_ki = ki * B;
        p.b_rs = B; p.b_ks = N * B;                     // other[(k*N + n)*B + b]
        p.c_mi = N * B; p.c_ni = B;                     // out[(m*N + n)*B + b]
        p.np2 = static_cast<int>(B);
        p.a_p2 = 1; p.b_p2 = 1; p.c_p2 = 1;
        p.alpha = inv_N;
        return launch_gemm(p, static_cast<hipStream_t>(stream), "outer_prod_mean_back_hip");
    };
    int rc = RC_OK;
    if (gleft)  rc = launch(right, gleft, D * L * L, L, L * L, 1);          // m = (d1,i), k = (d2,j)
    if (rc == RC_OK && gright) rc = launch(left, gright, L * L, 1, D * L * L, L);   // m = (d2,j), k = (d1,i)
    return rc;
}
