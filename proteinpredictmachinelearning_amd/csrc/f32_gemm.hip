// Binary32 contractions for gfx950: dense GEMM with bias (mul_mat), batched transposed GEMM with
// plane broadcast (out_prod, attention logits), outer-product-mean in both of the reference's layouts,
// triangle multiplication and the backward contractions of the last two.
//
// Reference behaviour restated here (paths relative to the reference tree):
//   mul_mat          src/backend/CPUKernels.cpp:763-771   (bias first, k ascending)
//   out_prod         src/backend/CPUKernels.cpp:787-887
//   outer_prod_mean  src/backend/CPUKernels.cpp:982-1032, src/ops/MathUtils.cpp:387-437
//
// Arithmetic.  Binary32 operands are multiplied on the bf16 matrix pipe through an exact three-way
// split (gemm_bf16x3_kernel, and gemm_planes_kernel for large problems, which splits ahead of the
// matrix work): products to within 2^-23 of |a||b|, sums in binary32, sixteen k per accumulation step,
// starting from bias[n] (or 0); alpha multiplies the finished sum.  Half operands go to the f16 matrix
// pipe unchanged (gemm_f16_kernel).  The clamped contraction of the triangle multiplication, whose
// result depends on how infinities propagate, stays on the fp32 pipe (gemm_f32_kernel:
// v_mfma_f32_32x32x2_f32, k ascending two at a time).
#include "common.hpp"

#include <atomic>
#include <type_traits>
#include <cstdlib>
#include <cstring>
#include <mutex>

namespace ppmlhip {
namespace {

constexpr int BM = 128, BN = 128, BK = 16;
constexpr int LDS_LD = BM + 4;        // row pitch of the k-major LDS tiles (floats)

enum LoadMode { LOAD_K_CONTIG = 0, LOAD_ROW_CONTIG = 1, LOAD_STRIDED = 2, LOAD_SPLIT_A = 4 };

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

// work-group -> (plane, tile row, tile col); bands of 8 tile rows keep operand panels in one L2
template <int TILE_M = BM>
__device__ __forceinline__ void tile_of_group(const GemmParams& p, int& plane, int& m0, int& n0) {
    const int tiles = p.tiles_m * p.tiles_n;
    const int total = tiles * p.np2 * p.np3;
    const int idx = xcd_contiguous_index(blockIdx.x, total);
    plane = idx / tiles;
    int t = idx - plane * tiles;
    const int band_rows = 8;
    const int band = t / (band_rows * p.tiles_n);
    t -= band * band_rows * p.tiles_n;
    const int rows_here = (p.tiles_m - band * band_rows) < band_rows ? (p.tiles_m - band * band_rows) : band_rows;
    const int tm = band * band_rows + t % rows_here;
    const int tn = t / rows_here;
    m0 = tm * TILE_M;
    n0 = tn * BN;
}

// The finished accumulators of one wave (TI x 2 tiles of 32 x 32) (rows from m_base, columns from n_base) go to C.
// CLAMP: the finite guard of the triangle multiplication (src/backend/CPUKernels.cpp:957-962): NaN -> 0,
// values beyond +-1e4 -> +-1e4.  A compile-time property: a run-time test in this store loop costs the
// other contractions a quarter of their speed.
template <bool SPLIT_C, bool STREAM_C, bool BIAS_LAST, bool CLAMP, int TI = 2>
__device__ __forceinline__ void store_acc(const GemmParams& p, float* __restrict__ C, const v16f (&acc)[TI][2],
                                          int m_base, int n_base, int lane) {
    const int j = lane & 31;
    const bool scale = p.alpha != 1.0f;
#pragma unroll
    for (int ti = 0; ti < TI; ++ti) {
        // The lane's sixteen rows of this tile are first + 8 * (r / 4) + r % 4.  With a compound row
        // index the quotient and remainder are formed once, for `first`, and stepped from there: a
        // division per element would cost more than the contraction itself on large outputs.
        const int first = m_base + ti * 32 + 4 * (lane >> 5);
        const int q0 = SPLIT_C ? first / p.c_lm : 0;
        const int r0 = SPLIT_C ? first - q0 * p.c_lm : 0;
        const bool one_wrap = p.c_lm >= 32;            // the sixteen rows span 28: at most one carry
#pragma unroll
        for (int tj = 0; tj < 2; ++tj) {
            const int n = n_base + tj * 32 + j;
            if (n >= p.N) continue;
            const float tail_bias = (BIAS_LAST && p.bias) ? p.bias[n] : 0.0f;
            int64_t coff;
            if (SPLIT_C) coff = static_cast<int64_t>(n / p.c_ln) * p.c_no + static_cast<int64_t>(n % p.c_ln) * p.c_ni;
            else         coff = static_cast<int64_t>(n) * p.c_ni;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int step = 8 * (r >> 2) + (r & 3);
                const int m = first + step;
                if (m >= p.M) continue;
                int64_t roff;
                if (SPLIT_C) {
                    int q = q0, rem = r0 + step;
                    if (one_wrap) { if (rem >= p.c_lm) { rem -= p.c_lm; ++q; } }
                    else { q += rem / p.c_lm; rem %= p.c_lm; }
                    roff = static_cast<int64_t>(q) * p.c_mo + static_cast<int64_t>(rem) * p.c_mi;
                } else {
                    roff = static_cast<int64_t>(m) * p.c_mi;
                }
                float v = acc[ti][tj][r];
                if (scale) v *= p.alpha;
                if (BIAS_LAST) v += tail_bias;
                if (CLAMP) v = (v != v) ? 0.0f : (v > 1e4f ? 1e4f : (v < -1e4f ? -1e4f : v));
                if (STREAM_C) __builtin_nontemporal_store(v, &C[roff + coff]);
                else C[roff + coff] = v;
            }
        }
    }
}

template <int MODE, bool SPLIT_C, bool STREAM_C, bool CLAMP = false>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const GemmParams p) {
    __shared__ __attribute__((aligned(16))) float lds_a[BK * LDS_LD];
    __shared__ __attribute__((aligned(16))) float lds_b[BK * LDS_LD];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int j = lane & 31, hh = lane >> 5;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;

    int plane, m0, n0;
    tile_of_group(p, plane, m0, n0);

    const int p2 = plane % p.np2, p3 = plane / p.np2;
    const float* A = p.A + p2 * p.a_p2 + p3 * p.a_p3;
    const float* B = p.B + (p2 / p.b_div2) * p.b_p2 + (p3 / p.b_div3) * p.b_p3;
    float* C = p.C + p2 * p.c_p2 + p3 * p.c_p3;

    v16f acc[2][2];
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) {
        const int n = n0 + wn + tj * 32 + j;
        const float b0 = (p.bias && n < p.N) ? p.bias[n] : 0.0f;
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

    store_acc<SPLIT_C, STREAM_C, false, CLAMP>(p, C, acc, m0 + wm, n0 + wn, lane);
}

// ------------------------------------------------------------------------------------------
// Many planes of small contractions with K <= 128 on the fp32 pipe (the triangle multiplication: 128 channel
// planes of 103 x 103 over K = 103).  With 128 x 128 tiles that is one work-group per plane, half the CUs idle, each
// walking seven 16-k stages of load -> LDS -> 32 MFMAs per wave -> barrier one after the other.  Here a work-group
// takes a 64 x 64 tile (four per plane: every CU has two), loads the whole K of both panels at once -- one memory
// round trip -- and then runs its K / 2 MFMAs per wave out of LDS without a barrier in between.  Products and sums are
// those of gemm_f32_kernel in the same order (k ascending two at a time from the bias): same bits.
constexpr int MIDK_MAX = 128;
template <int MODE> struct MidK { static constexpr int LD = MODE == LOAD_ROW_CONTIG ? 68 : 65; };   // floats per k row of a panel

template <int MODE, bool CLAMP>
__global__ __launch_bounds__(256) void gemm_f32_midk_kernel(const GemmParams p, int kp) {
    static_assert(MODE == LOAD_K_CONTIG || MODE == LOAD_ROW_CONTIG, "contiguous operands only");
    constexpr int T = 64, LD = MidK<MODE>::LD;
    extern __shared__ __attribute__((aligned(16))) float lds_midk[];
    float* const lds_a = lds_midk;                      // [kp][LD]: k-major, rows contiguous
    float* const lds_b = lds_midk + kp * LD;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int j = lane & 31, hh = lane >> 5;
    const int wm = (wave >> 1) * 32, wn = (wave & 1) * 32;
    const int tiles_m = (p.M + T - 1) / T, tiles_n = (p.N + T - 1) / T;
    const int tiles = tiles_m * tiles_n;
    const int idx = xcd_contiguous_index(blockIdx.x, tiles * p.np2 * p.np3);
    const int plane = idx / tiles;
    const int t = idx - plane * tiles;
    const int m0 = (t / tiles_n) * T, n0 = (t % tiles_n) * T;
    const int p2 = plane % p.np2, p3 = plane / p.np2;
    const float* A = p.A + p2 * p.a_p2 + p3 * p.a_p3;
    const float* B = p.B + (p2 / p.b_div2) * p.b_p2 + (p3 / p.b_div3) * p.b_p3;
    float* C = p.C + p2 * p.c_p2 + p3 * p.c_p3;

    // ---- both panels, all of K, in flight at once
    v4f ra[8], rb[8];
    const auto load_panel = [&](const float* __restrict__ base, int64_t rs, int64_t ks, int row0, int nrows, v4f (&reg)[8]) {
#pragma unroll
        for (int it = 0; it < 8; ++it) {
            v4f v = {0.f, 0.f, 0.f, 0.f};
            if (MODE == LOAD_K_CONTIG) {
                // sixteen lanes along 64 k of a row, four rows per wave instruction
                const int row = row0 + (tid >> 4) + 16 * (it & 3);
                const int k = (tid & 15) * 4 + 64 * (it >> 2);
                if (row < nrows && k < p.K) {
                    const float* src = base + static_cast<int64_t>(row) * rs + k;
                    if (k + 3 < p.K) v = *reinterpret_cast<const v4f_u*>(src);
                    else {
#pragma unroll
                        for (int c = 0; c < 4; ++c) if (k + c < p.K) v[c] = src[c];
                    }
                }
            } else {
                // sixteen lanes along the 64 rows of one k, four k per wave instruction
                const int k = (tid >> 4) + 16 * it;
                const int row = row0 + (tid & 15) * 4;
                if (k < p.K && row < nrows) {
                    const float* src = base + static_cast<int64_t>(k) * ks + row;
                    if (row + 3 < nrows) v = *reinterpret_cast<const v4f_u*>(src);
                    else {
#pragma unroll
                        for (int c = 0; c < 4; ++c) if (row + c < nrows) v[c] = src[c];
                    }
                }
            }
            reg[it] = v;
        }
    };
    const auto park_panel = [&](float* __restrict__ lds, const v4f (&reg)[8]) {
#pragma unroll
        for (int it = 0; it < 8; ++it) {
            if (MODE == LOAD_K_CONTIG) {
                const int row = (tid >> 4) + 16 * (it & 3);
                const int k = (tid & 15) * 4 + 64 * (it >> 2);
#pragma unroll
                for (int c = 0; c < 4; ++c) if (k + c < kp) lds[(k + c) * LD + row] = reg[it][c];
            } else {
                const int k = (tid >> 4) + 16 * it;
                if (k < kp) *reinterpret_cast<v4f*>(lds + k * LD + (tid & 15) * 4) = reg[it];
            }
        }
    };
    load_panel(A, p.a_rs, p.a_ks, m0, p.M, ra);
    load_panel(B, p.b_rs, p.b_ks, n0, p.N, rb);

    v16f acc;
    {
        const int n = n0 + wn + j;
        const float b0 = (p.bias && n < p.N) ? p.bias[n] : 0.0f;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = b0;
    }
    park_panel(lds_a, ra);
    park_panel(lds_b, rb);
    __syncthreads();

    const float* fa = lds_a + hh * LD + wm + j;
    const float* fb = lds_b + hh * LD + wn + j;
    int kk = 0;
    for (; kk + 16 <= kp; kk += 16) {                   // eight steps' operands are read ahead of their MFMAs
        float a[8], b[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) { a[u] = fa[(kk + 2 * u) * LD]; b[u] = fb[(kk + 2 * u) * LD]; }
#pragma unroll
        for (int u = 0; u < 8; ++u) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u], b[u], acc, 0, 0, 0);
    }
    for (; kk < kp; kk += 2) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[kk * LD], fb[kk * LD], acc, 0, 0, 0);

    const int n = n0 + wn + j;
    if (n >= p.N) return;
    const bool scale = p.alpha != 1.0f;
    float* out = C + static_cast<int64_t>(n) * p.c_ni;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm + 4 * hh + 8 * (r >> 2) + (r & 3);
        if (m >= p.M) continue;
        float v = acc[r];
        if (scale) v *= p.alpha;
        if (CLAMP) v = (v != v) ? 0.0f : (v > 1e4f ? 1e4f : (v < -1e4f ? -1e4f : v));
        out[static_cast<int64_t>(m) * p.c_mi] = v;
    }
}

template <int MODE, bool CLAMP>
int launch_f32_midk(const GemmParams& p, hipStream_t stream, const char* what) {
    const int kp = (p.K + 1) & ~1;
    const size_t lds = static_cast<size_t>(2) * kp * MidK<MODE>::LD * sizeof(float);
    auto kernel = &gemm_f32_midk_kernel<MODE, CLAMP>;
    // more than 64 KB of dynamic LDS has to be asked for, once per instance and device
    constexpr int MAX_DEVICES = 64;
    static std::atomic<bool> sized[MAX_DEVICES];
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); dev = -1; }
    const bool known = dev >= 0 && dev < MAX_DEVICES;
    if (!known || !sized[dev].load(std::memory_order_acquire)) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                2 * MIDK_MAX * MidK<MODE>::LD * static_cast<int>(sizeof(float))) != hipSuccess) {
            (void)hipGetLastError();
            set_error("%s: cannot size the LDS of the whole-K kernel", what);
            return RC_LAUNCH;
        }
        if (known) sized[dev].store(true, std::memory_order_release);
    }
    const int64_t tiles = static_cast<int64_t>((p.M + 63) / 64) * ((p.N + 63) / 64) * p.np2 * p.np3;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(tiles)), dim3(256), lds, stream, p, kp);
    return check_launch(what);
}

// ------------------------------------------------------------------------------------------
// The same contraction on the bf16 matrix pipe, whose rate is sixteen times that of the fp32 one (which,
// moreover, never runs beside vector instructions on this chip).  A binary32 number is the exact sum of three bf16 numbers
// (x = x1 + x2 + x3: 8 + 8 + 8 significant bits, taken off the top by truncation), so a product is
// the exact sum of nine bf16 x bf16 products, each of which the matrix pipe forms exactly and adds
// into a binary32 accumulator.  Six of them are kept -- (1,1) (1,2) (2,1) (1,3) (3,1) (2,2) -- and the
// three dropped ones are below 2^-23 of |a||b| together, i.e. about one rounding of a binary32
// product; the accumulation itself is binary32 as before.  What differs from the fp32 pipe is the
// order of the roundings inside a group of 16 k, not their size.
// Operands the three parts cannot carry -- non-finite ones (x - x1 is NaN for an infinite x) and ones whose lower
// parts fall below bf16's smallest step 2^-133 -- are noticed while they are split (SplitGuard, common.hpp), and the
// outputs they touch are redone by plain_dot() below in plain binary32 arithmetic, the reference's own loop: the
// split pipe then gives +-inf where the reference does and keeps every bit of a subnormal operand.  The clamped
// instances stay on the fp32 pipe.
constexpr int SPLIT_PITCH = 48;                   // bytes per tile row in a plane: 16 bf16, then 16 bytes of padding
constexpr int SPLIT_PLANE = BM * SPLIT_PITCH;     // one of the three bf16 planes of a 128 x 16 operand tile

// One output the reference's way (src/backend/CPUKernels.cpp:763-771, 836-884, 1006-1028): from the bias (or zero),
// one product at a time, k ascending, every product and every sum rounded to binary32 on its own (this file is
// compiled without contraction).  A and B are the plane's bases.
__device__ __forceinline__ float plain_dot(const GemmParams& p, const float* __restrict__ A, const float* __restrict__ B, int m, int n) {
    float s = p.bias ? p.bias[n] : 0.0f;
    const int64_t ra = p.a_lm > 0 ? static_cast<int64_t>(m / p.a_lm) * p.a_mo + static_cast<int64_t>(m % p.a_lm) * p.a_mi
                                  : static_cast<int64_t>(m) * p.a_rs;
    const float* b = B + static_cast<int64_t>(n) * p.b_rs;
    for (int k = 0; k < p.K; ++k) {
        const float a = p.a_lm > 0 ? A[ra + static_cast<int64_t>(k / p.a_lk) * p.a_ko + static_cast<int64_t>(k % p.a_lk) * p.a_ki]
                                   : A[ra + static_cast<int64_t>(k) * p.a_ks];
        const float prod = a * b[static_cast<int64_t>(k) * p.b_ks];
        s = s + prod;
    }
    return s;
}

// A whole tile of the output (rows x cols from (m0, n0) of the plane whose bases are A, B, C) by plain_dot, written
// straight to C with the contraction's own output addressing: what a work-group does INSTEAD of storing its
// accumulators when a SplitGuard fired for the tile.  One loop, no use of the accumulators: the ordinary path pays
// nothing for it but the test.
__device__ __forceinline__ void plain_tile(const GemmParams& p, const float* __restrict__ A, const float* __restrict__ B,
                                           float* __restrict__ C, int m0, int n0, int rows, int cols, int tid) {
    for (int e = tid; e < rows * cols; e += 256) {
        const int m = m0 + e / cols, n = n0 + e % cols;
        if (m >= p.M || n >= p.N) continue;
        const float v = plain_dot(p, A, B, m, n) * p.alpha;
        C[static_cast<int64_t>(m / p.c_lm) * p.c_mo + static_cast<int64_t>(m % p.c_lm) * p.c_mi +
          static_cast<int64_t>(n / p.c_ln) * p.c_no + static_cast<int64_t>(n % p.c_ln) * p.c_ni] = v;
    }
}

// The same for the kernels whose operands have contiguous rows (A(m, k) = A[k * a_ks + m]) and whose output plane is
// dense (C[m * ldc + n]), without bias: it names nothing that those kernels do not hold already.
__device__ __forceinline__ void plain_tile_rows(const float* __restrict__ A, const float* __restrict__ B, float* __restrict__ C,
                                                int a_ks, int b_ks, int ldc, int K, float alpha, int M, int N,
                                                int m0, int n0, int side, int tid) {
    for (int e = tid; e < side * side; e += 256) {
        const int m = m0 + e / side, n = n0 + e % side;      // (side is a power of two)
        if (m >= M || n >= N) continue;
        float s = 0.0f;
        for (int k = 0; k < K; ++k) {
            const float prod = A[static_cast<int64_t>(k) * a_ks + m] * B[static_cast<int64_t>(k) * b_ks + n];
            s = s + prod;
        }
        C[static_cast<int64_t>(m) * ldc + n] = s * alpha;
    }
}

// Tile `t` of the short-K kernel's tile list (tiles of `side` x `side`, planes laid end to end) by plain_tile_rows, with
// every parameter read afresh from the kernel-argument segment, where the launch's GemmParams lies first: the ordinary
// path then holds nothing alive for this one (held in registers across the tile loop, the few pointers and sizes it
// needs cost that loop a third of a microsecond per launch in scheduling freedom).
__device__ __forceinline__ void shortk_tile_again_inline(int t, int side, int tid) {
#if defined(__HIP_DEVICE_COMPILE__)                     // (the host pass of this file knows neither the builtin nor its address space)
    typedef const __attribute__((address_space(4))) GemmParams* KernargParams;
    KernargParams q = (KernargParams)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(q));                         // not the same values as the kernel's own copy, as far as the compiler knows
#else
    const GemmParams* q = nullptr;
#endif
    const int tiles_m = (q->M + side - 1) / side, tiles_n = (q->N + side - 1) / side;
    const int plane = t / (tiles_m * tiles_n);
    const int r = t - plane * tiles_m * tiles_n;
    const int p2 = plane % q->np2, p3 = plane / q->np2;
    const float* A = q->A + p2 * q->a_p2 + p3 * q->a_p3;
    const float* B = q->B + (p2 / q->b_div2) * q->b_p2 + (p3 / q->b_div3) * q->b_p3;
    float* C = q->C + p2 * q->c_p2 + p3 * q->c_p3;
    plain_tile_rows(A, B, C, static_cast<int>(q->a_ks), static_cast<int>(q->b_ks), static_cast<int>(q->c_mi), q->K, q->alpha, q->M, q->N,
                    (r / tiles_n) * side, (r % tiles_n) * side, side, tid);
}

// What a work-group of the short-K kernel does once its tile loop has ended, if a SplitGuard fired in it: bit i of
// `fired_its` stands for the i-th tile the work-group took (bit 63 for that one and every later one), and those tiles
// are written again by shortk_tile_again_inline.  The work-group's tile list is rebuilt from the kernel-argument
// segment (`total_tiles` follows the GemmParams there) and its own number, exactly as the kernel builds it.
__device__ __forceinline__ void shortk_redo_fired(uint64_t fired_its, int side, int tid) {
#if defined(__HIP_DEVICE_COMPILE__)
    typedef const __attribute__((address_space(4))) int* KernargInt;
    KernargInt words = (KernargInt)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(words));
    static_assert(sizeof(GemmParams) % 8 == 0, "the next kernel argument follows the structure without padding");
    const int total_tiles = words[sizeof(GemmParams) / 4];
#else
    const int total_tiles = 0;
#endif
    constexpr int XCDS = 8;
    const int groups = static_cast<int>(gridDim.x) / XCDS;
    const int xcd = static_cast<int>(blockIdx.x) % XCDS, slot = static_cast<int>(blockIdx.x) / XCDS;
    const int part = (total_tiles + XCDS - 1) / XCDS;
    const int part_begin = xcd * part;
    const int part_end = part_begin + part < total_tiles ? part_begin + part : total_tiles;
    int i = 0;
    for (int t = part_begin + slot; t < part_end; t += groups, ++i)
        if ((fired_its >> (i < 63 ? i : 63)) & 1) shortk_tile_again_inline(t, side, tid);
}

// A thread's share of a 128 x 16 operand tile goes to the planes.  Operands with contiguous rows are
// read one row and eight consecutive k per thread (eight loads, each contiguous across the lanes), the
// others two rows and four consecutive k each.
template <int MODE>
__device__ __forceinline__ void split_store(uint8_t* __restrict__ planes, int tid, const v4f (&reg)[2], SplitGuard& guard) {
    uint2 lo[3], hi[3];
    split4(reg[0], lo, guard);
    split4(reg[1], hi, guard);
    if (MODE == LOAD_ROW_CONTIG) {
        uint8_t* dst = planes + (tid & 127) * SPLIT_PITCH + (tid >> 7) * 16;
#pragma unroll
        for (int s = 0; s < 3; ++s) *reinterpret_cast<uint4*>(dst + s * SPLIT_PLANE) = uint4{lo[s].x, lo[s].y, hi[s].x, hi[s].y};
    } else {
        uint8_t* dst = planes + (tid >> 2) * SPLIT_PITCH + (tid & 3) * 8;
#pragma unroll
        for (int s = 0; s < 3; ++s) {
            *reinterpret_cast<uint2*>(dst + s * SPLIT_PLANE) = lo[s];
            *reinterpret_cast<uint2*>(dst + s * SPLIT_PLANE + 64 * SPLIT_PITCH) = hi[s];
        }
    }
}

// one row, eight consecutive k of an operand whose rows are contiguous in memory: A(row, k) = base[k * ks + row]
__device__ __forceinline__ void load_rows8(const float* __restrict__ base, int64_t ks, int row0, int nrows, int k0, int K,
                                           int tid, v4f (&reg)[2]) {
    const int row = row0 + (tid & 127);
    const int kb = k0 + (tid >> 7) * 8;
    const float* src = base + static_cast<int64_t>(kb) * ks + row;
#pragma unroll
    for (int c = 0; c < 8; ++c)
        reg[c >> 2][c & 3] = (row < nrows && kb + c < K) ? src[static_cast<int64_t>(c) * ks] : 0.0f;
}

// ---- buffer-addressed forms for planes below 2 GiB (FAST_IO).  The generic paths above spend most of the
// kernel's vector instructions on 64-bit address arithmetic and bounds tests (counters at the attention-logit
// shapes: about 1150 vector instructions per wave, of which the split is 180); a buffer resource per plane
// takes both over: the address is one 32-bit add per access, and an access whose offset is not inside the
// plane is dropped (stores) or returns zero (loads) in hardware.  Lanes whose row or column lies outside the
// matrix carry an offset of 2^31, which no plane reaches.
constexpr uint32_t OUTSIDE = 0x80000000u;

// one row, eight consecutive k of an operand plane [K][ks] whose rows are contiguous: A(row, k) = plane[k * ks + row]
__device__ __forceinline__ void load_rows8_buffer(const __amdgpu_buffer_rsrc_t rsrc, uint32_t ks_bytes, int row0, int nrows, int k0,
                                                  int tid, v4f (&reg)[2]) {
    const int row = row0 + (tid & 127);
    const uint32_t lane_off = row < nrows ? static_cast<uint32_t>(row) * 4u : OUTSIDE;
    // k is the same for the whole wave: its part of the offset is scalar arithmetic
    const uint32_t kb = static_cast<uint32_t>(k0 + __builtin_amdgcn_readfirstlane(tid >> 7) * 8);
#pragma unroll
    for (int c = 0; c < 8; ++c)
        reg[c >> 2][c & 3] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, lane_off + (kb + c) * ks_bytes, 0, 0));
}

// two rows (tid / 4 and tid / 4 + 64 of the tile), four consecutive k each, of an operand plane whose rows are
// contiguous in k: A(row, k) = plane[row * rs + k].  K4 (K a multiple of four): a piece of sixteen bytes never runs
// over the end of its row, so it is one load; otherwise element by element.  No branch either way: the generic form
// of this load sits inside tests of the row and of the row's end, and the compiler waits for every load at the end of
// its branch (26368 x 256 -> 256: 29 us, the waves waiting 38 % of it; 25 us with this form).
template <bool K4>
__device__ __forceinline__ void load_kcontig_buffer(const __amdgpu_buffer_rsrc_t rsrc, uint32_t rs_bytes, int row0, int nrows, int k0, int K,
                                                    int tid, v4f (&reg)[2]) {
    const int k = k0 + (tid & 3) * 4;
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        const int row = row0 + (tid >> 2) + it * 64;
        const uint32_t at = row < nrows ? static_cast<uint32_t>(row) * rs_bytes + static_cast<uint32_t>(k) * 4u : OUTSIDE;
        if (K4) {
            const v4i raw = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc, k < K ? at : OUTSIDE, 0, 0));
            reg[it] = __builtin_bit_cast(v4f, raw);
        } else {
#pragma unroll
            for (int c = 0; c < 4; ++c)
                reg[it][c] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, k + c < K ? at + 4u * c : OUTSIDE, 0, 0));
        }
    }
}

// The finished accumulators of one wave to a dense plane C[m * ld + n] through a buffer resource over the plane.
// (TAIL: tail[tj] joins the finished sums of the lane's column in tile column tj -- a bias that is added last; the
// caller has loaded it long before: a load here would be waited for with a count that every earlier store is part of)
template <bool STREAM_C, bool TAIL = false>
__device__ __forceinline__ void store_acc_buffer(const __amdgpu_buffer_rsrc_t rsrc, uint32_t ld_bytes, int N, float alpha,
                                                 const v16f (&acc)[2][2], int m_base, int n_base, int lane,
                                                 float tail0 = 0.0f, float tail1 = 0.0f) {
    const int j = lane & 31;
    const bool scale = alpha != 1.0f;
#pragma unroll
    for (int ti = 0; ti < 2; ++ti) {
        const uint32_t first = static_cast<uint32_t>(m_base + ti * 32 + 4 * (lane >> 5));
#pragma unroll
        for (int tj = 0; tj < 2; ++tj) {
            const int n = n_base + tj * 32 + j;
            // rows past the matrix fall outside the plane by themselves (offset >= M * ld bytes)
            const uint32_t base = n < N ? first * ld_bytes + static_cast<uint32_t>(n) * 4u : OUTSIDE;
            const float tail = tj ? tail1 : tail0;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float v = acc[ti][tj][r];
                if (scale) v *= alpha;
                if (TAIL) v += tail;
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), rsrc, base + (8 * (r >> 2) + (r & 3)) * ld_bytes, 0,
                                                      STREAM_C ? 3 : 0);
            }
        }
    }
}

template <int MODE, bool SPLIT_C, bool STREAM_C, bool FAST_IO = false, bool K4 = true>
__global__ __launch_bounds__(256) void gemm_bf16x3_kernel(const GemmParams p) {
    // (FAST_IO with SPLIT_C: buffer-addressed loads, the output by its compound addressing)
    static_assert(!FAST_IO || MODE == LOAD_ROW_CONTIG || MODE == LOAD_K_CONTIG, "buffer addressing: rows contiguous in themselves or in k");
    __shared__ __attribute__((aligned(16))) uint8_t lds_a[3 * SPLIT_PLANE];
    __shared__ __attribute__((aligned(16))) uint8_t lds_b[3 * SPLIT_PLANE];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int j = lane & 31, hh = lane >> 5;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;

    int plane, m0, n0;
    tile_of_group(p, plane, m0, n0);
    const int p2 = plane % p.np2, p3 = plane / p.np2;
    const float* A = p.A + p2 * p.a_p2 + p3 * p.a_p3;
    const float* B = p.B + (p2 / p.b_div2) * p.b_p2 + (p3 / p.b_div3) * p.b_p3;
    float* C = p.C + p2 * p.c_p2 + p3 * p.c_p3;

    v16f acc[2][2];
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) {
        const int n = n0 + wn + tj * 32 + j;
        const float b0 = (p.bias && n < p.N) ? p.bias[n] : 0.0f;
#pragma unroll
        for (int ti = 0; ti < 2; ++ti)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[ti][tj][r] = b0;
    }

    v4f ra[2], rb[2];
    constexpr int MODE_B = MODE == LOAD_SPLIT_A ? LOAD_STRIDED : MODE;
    // FAST_IO: one buffer resource per operand plane and for the output plane (sizes checked by the launcher)
    __amdgpu_buffer_rsrc_t rsrc_a, rsrc_b, rsrc_c;
    if (FAST_IO) {
        const int64_t a_plane = MODE == LOAD_K_CONTIG ? (p.M - 1) * p.a_rs + p.K : p.K * p.a_ks;     // floats from the plane's base to its end
        const int64_t b_plane = MODE == LOAD_K_CONTIG ? (p.N - 1) * p.b_rs + p.K : p.K * p.b_ks;
        rsrc_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(A), 0, static_cast<int>(a_plane * 4), 0x00020000);
        rsrc_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(B), 0, static_cast<int>(b_plane * 4), 0x00020000);
        if (!SPLIT_C) rsrc_c = __builtin_amdgcn_make_buffer_rsrc(C, 0, static_cast<int>(p.M * p.c_mi * 4), 0x00020000);
    }
    const auto load_both = [&](int k0) {
        if (FAST_IO && MODE == LOAD_K_CONTIG) {
            load_kcontig_buffer<K4>(rsrc_a, static_cast<uint32_t>(p.a_rs) * 4u, m0, p.M, k0, p.K, tid, ra);
            load_kcontig_buffer<K4>(rsrc_b, static_cast<uint32_t>(p.b_rs) * 4u, n0, p.N, k0, p.K, tid, rb);
        } else if (FAST_IO) {
            load_rows8_buffer(rsrc_a, static_cast<uint32_t>(p.a_ks) * 4u, m0, p.M, k0, tid, ra);
            load_rows8_buffer(rsrc_b, static_cast<uint32_t>(p.b_ks) * 4u, n0, p.N, k0, tid, rb);
        } else if (MODE == LOAD_ROW_CONTIG) {
            load_rows8(A, p.a_ks, m0, p.M, k0, p.K, tid, ra);
            load_rows8(B, p.b_ks, n0, p.N, k0, p.K, tid, rb);
        } else {
            if (MODE == LOAD_SPLIT_A) load_tile_split(A, p, m0, p.M, k0, p.K, tid, ra);
            else load_tile<MODE>(A, p.a_rs, p.a_ks, m0, p.M, k0, p.K, tid, ra);
            load_tile<MODE_B>(B, p.b_rs, p.b_ks, n0, p.N, k0, p.K, tid, rb);
        }
    };
    load_both(0);

    // a lane's fragment of a plane: its row's k = 8 * hh .. 8 * hh + 7, sixteen bytes
    const uint8_t* frag_a = lds_a + (wm + j) * SPLIT_PITCH + hh * 16;
    const uint8_t* frag_b = lds_b + (wn + j) * SPLIT_PITCH + hh * 16;

    SplitGuard guard;
    for (int k0 = 0; k0 < p.K; k0 += BK) {
        split_store<MODE>(lds_a, tid, ra, guard);
        split_store<MODE>(lds_b, tid, rb, guard);
        __syncthreads();
        if (k0 + BK < p.K) load_both(k0 + BK);
        v8bf fa[2][3], fb[2][3];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int s = 0; s < 3; ++s) {
                fa[t][s] = *reinterpret_cast<const v8bf*>(frag_a + s * SPLIT_PLANE + t * 32 * SPLIT_PITCH);
                fb[t][s] = *reinterpret_cast<const v8bf*>(frag_b + s * SPLIT_PLANE + t * 32 * SPLIT_PITCH);
            }
#pragma unroll
        for (int q = 0; q < 6; ++q)
#pragma unroll
            for (int ti = 0; ti < 2; ++ti)
#pragma unroll
                for (int tj = 0; tj < 2; ++tj)
                    acc[ti][tj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[ti][SPLIT_TERMS[q][0]], fb[tj][SPLIT_TERMS[q][1]], acc[ti][tj], 0, 0, 0);
        __syncthreads();
    }

    // an operand of this tile that the split could not carry (non-finite, or bits below 2^-133): the whole tile again,
    // the reference's way
    if (__syncthreads_or(guard.fired() ? 1 : 0)) {
        plain_tile(p, A, B, C, m0, n0, BM, BN, tid);
        return;
    }

    if (FAST_IO && !SPLIT_C) store_acc_buffer<STREAM_C>(rsrc_c, static_cast<uint32_t>(p.c_mi) * 4u, p.N, p.alpha, acc, m0 + wm, n0 + wn, lane);
    else store_acc<SPLIT_C, STREAM_C, false, false>(p, C, acc, m0 + wm, n0 + wn, lane);
}

// ------------------------------------------------------------------------------------------
// The same contraction with the work of a work-group divided between two sets of waves.  In gemm_bf16x3_kernel a wave
// splits its share of a 16-k chunk (vector pipe), waits at a barrier, and then issues the chunk's matrix work (matrix
// pipe): with at most one work-group per CU -- a LinearLayer-shaped contraction of a few hundred tiles, or a small
// square one -- the two pipes take turns and the K loop costs 1.2 us per chunk whatever the problem's size
// (408 x 256 -> 16 and 26368 x 256 -> 128 both took 19 to 20 us).  Here waves 4..7 of a work-group of eight only load
// and split (chunk k + 1, into the other half of a double buffer, from loads issued three chunks ahead: they hold no
// accumulators, so the registers are there), and waves 0..3 only read fragments and issue MFMAs (chunk k); one barrier
// per chunk.  Every SIMD hosts one wave of each kind, so the vector and the matrix pipe work at the same time.  Same
// thread-to-element mapping, same fragments, same order of the products as gemm_bf16x3_kernel: same bits.  Buffer
// addressing throughout (the launcher's conditions for it).  Measured, us, this / gemm_bf16x3_kernel: 408 x 256 -> 16
// 13.5 / 19.1, 26368 x 256 -> 16 .. 128 15.0 - 16.9 / 20.3, 10609 x 256 -> 128 14.7 / 19.6, 1024^3 41 / 65; with
// more tiles than CUs (26368 x 256 -> 256 and wider, the many-plane contractions) the work-groups of a CU overlap
// each other anyway and the two forms measure the same: the launcher takes this one up to one tile per CU.
constexpr int PC_AHEAD = 3;                       // chunks a producer wave has in flight
template <int MODE, bool STREAM_C, bool K4, int BMODE = MODE>
__global__ __launch_bounds__(512) void gemm_bf16x3_pc_kernel(const GemmParams p) {
    // (MODE: how A lies; BMODE: how B lies -- the backward of the triangle multiplication contracts a gradient that is
    // contiguous in k with an operand that is contiguous in its rows)
    static_assert(MODE == LOAD_ROW_CONTIG || MODE == LOAD_K_CONTIG, "buffer addressing");
    static_assert(BMODE == LOAD_ROW_CONTIG || BMODE == LOAD_K_CONTIG, "buffer addressing");
    constexpr int STAGE = 3 * SPLIT_PLANE;            // the three planes of one operand's chunk
    __shared__ __attribute__((aligned(16))) uint8_t lds_ab[2][2 * STAGE];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 31, hh = lane >> 5;
    const bool producer = wave >= 4;
    const int ptid = tid & 255;                         // a producer's number in gemm_bf16x3_kernel's thread-to-element mapping
    const int cw = wave & 3;
    const int wm = (cw >> 1) * 64, wn = (cw & 1) * 64;

    int plane, m0, n0;
    tile_of_group(p, plane, m0, n0);
    const int p2 = plane % p.np2, p3 = plane / p.np2;
    const float* A = p.A + p2 * p.a_p2 + p3 * p.a_p3;
    const float* B = p.B + (p2 / p.b_div2) * p.b_p2 + (p3 / p.b_div3) * p.b_p3;
    float* C = p.C + p2 * p.c_p2 + p3 * p.c_p3;
    const int chunks = (p.K + BK - 1) / BK;

    const int64_t a_plane = MODE == LOAD_K_CONTIG ? (p.M - 1) * p.a_rs + p.K : p.K * p.a_ks;
    const int64_t b_plane = BMODE == LOAD_K_CONTIG ? (p.N - 1) * p.b_rs + p.K : p.K * p.b_ks;
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(A), 0, static_cast<int>(a_plane * 4), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(B), 0, static_cast<int>(b_plane * 4), 0x00020000);

    // Both kinds of wave pass chunks + 1 barriers in their loops: barrier i + 1 says "chunk i is in LDS" and "chunk
    // i - 1 has been read".
    int fired = 0;
    if (producer) {
        v4f ra[PC_AHEAD][2], rb[PC_AHEAD][2];
        const auto load_both = [&](int c, v4f (&xa)[2], v4f (&xb)[2]) {
            if (MODE == LOAD_K_CONTIG) load_kcontig_buffer<K4>(rsrc_a, static_cast<uint32_t>(p.a_rs) * 4u, m0, p.M, c * BK, p.K, ptid, xa);
            else load_rows8_buffer(rsrc_a, static_cast<uint32_t>(p.a_ks) * 4u, m0, p.M, c * BK, ptid, xa);
            if (BMODE == LOAD_K_CONTIG) load_kcontig_buffer<K4>(rsrc_b, static_cast<uint32_t>(p.b_rs) * 4u, n0, p.N, c * BK, p.K, ptid, xb);
            else load_rows8_buffer(rsrc_b, static_cast<uint32_t>(p.b_ks) * 4u, n0, p.N, c * BK, ptid, xb);
        };
#pragma unroll
        for (int d = 0; d < PC_AHEAD; ++d)
            if (d < chunks) load_both(d, ra[d], rb[d]);
        SplitGuard guard;
        // chunk c goes to half c % 2 while the other waves contract chunk c - 1 out of the other half; the register
        // sets take turns by name (the loop body is written out PC_AHEAD times)
        for (int cg = 0; cg < chunks; cg += PC_AHEAD) {
#pragma unroll
            for (int d = 0; d < PC_AHEAD; ++d) {
                const int c = cg + d;
                if (c >= chunks) break;                 // uniform
                uint8_t* half = lds_ab[c & 1];
                split_store<MODE>(half, ptid, ra[d], guard);
                split_store<BMODE>(half + STAGE, ptid, rb[d], guard);
                if (c + PC_AHEAD < chunks) load_both(c + PC_AHEAD, ra[d], rb[d]);
                __syncthreads();
            }
        }
        __syncthreads();                                // (the other waves' last chunk)
        fired = guard.fired() ? 1 : 0;
    }

    v16f acc[2][2];
    if (!producer) {
#pragma unroll
        for (int tj = 0; tj < 2; ++tj) {
            const int n = n0 + wn + tj * 32 + j;
            const float b0 = (p.bias && n < p.N) ? p.bias[n] : 0.0f;
#pragma unroll
            for (int ti = 0; ti < 2; ++ti)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[ti][tj][r] = b0;
        }
        const int frag_a = (wm + j) * SPLIT_PITCH + hh * 16;
        const int frag_b = STAGE + (wn + j) * SPLIT_PITCH + hh * 16;
        __syncthreads();                                // chunk 0 is in LDS
        for (int c = 0; c < chunks; ++c) {
            const uint8_t* half = lds_ab[c & 1];
            v8bf fa[2][3], fb[2][3];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int s = 0; s < 3; ++s) {
                    fa[t][s] = *reinterpret_cast<const v8bf*>(half + frag_a + s * SPLIT_PLANE + t * 32 * SPLIT_PITCH);
                    fb[t][s] = *reinterpret_cast<const v8bf*>(half + frag_b + s * SPLIT_PLANE + t * 32 * SPLIT_PITCH);
                }
#pragma unroll
            for (int q = 0; q < 6; ++q)
#pragma unroll
                for (int ti = 0; ti < 2; ++ti)
#pragma unroll
                    for (int tj = 0; tj < 2; ++tj)
                        acc[ti][tj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[ti][SPLIT_TERMS[q][0]], fb[tj][SPLIT_TERMS[q][1]], acc[ti][tj], 0, 0, 0);
            __syncthreads();                            // chunk c has been read; chunk c + 1 is in LDS
        }
    }

    // an operand of this tile that the split could not carry: the whole tile again, the reference's way
    if (__syncthreads_or(fired)) {
        if (tid < 256) plain_tile(p, A, B, C, m0, n0, BM, BN, tid);
        return;
    }
    if (!producer) {
        const __amdgpu_buffer_rsrc_t rsrc_c = __builtin_amdgcn_make_buffer_rsrc(C, 0, static_cast<int>(p.M * p.c_mi * 4), 0x00020000);
        store_acc_buffer<STREAM_C>(rsrc_c, static_cast<uint32_t>(p.c_mi) * 4u, p.N, p.alpha, acc, m0 + wm, n0 + wn, lane);
    }
}

// gemm_bf16x3_pc_kernel for a few output tiles under a long K (a LinearLayer's weight gradient: 256 x 768 outputs over
// 26368 tokens -- twelve tiles): the K loop is cut into slices, one work-group per (tile, slice) -- the tile numbering
// takes the slice for the plane --, raw sums go to partial[slice][m][n] and reduce_slices_kernel adds them in slice
// order, applies bias, factor and the output's addressing.  A slice whose split could not carry an operand leaves NaN
// for its whole tile, and reduce_slices_kernel computes every output whose sum is NaN the reference's way (no flags to
// clear ahead: one launch less).
template <int MODE, bool K4>
__global__ __launch_bounds__(512) void gemm_bf16x3_pc_slices_kernel(const GemmParams p, int chunks, int slice_chunks, float* __restrict__ partial,
                                                                    int ma_pad, int nb_pad) {
    static_assert(MODE == LOAD_ROW_CONTIG || MODE == LOAD_K_CONTIG, "buffer addressing");
    constexpr int STAGE = 3 * SPLIT_PLANE;
    __shared__ __attribute__((aligned(16))) uint8_t lds_ab[2][2 * STAGE];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 31, hh = lane >> 5;
    const bool producer = wave >= 4;
    const int ptid = tid & 255;
    const int cw = wave & 3;
    const int wm = (cw >> 1) * 64, wn = (cw & 1) * 64;

    int slice, m0, n0;
    tile_of_group(p, slice, m0, n0);
    const int c_begin = slice * slice_chunks;
    const int c_end = c_begin + slice_chunks < chunks ? c_begin + slice_chunks : chunks;
    const int nch = c_end - c_begin;

    const int64_t a_plane = MODE == LOAD_K_CONTIG ? (p.M - 1) * p.a_rs + p.K : p.K * p.a_ks;
    const int64_t b_plane = MODE == LOAD_K_CONTIG ? (p.N - 1) * p.b_rs + p.K : p.K * p.b_ks;
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.A), 0, static_cast<int>(a_plane * 4), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.B), 0, static_cast<int>(b_plane * 4), 0x00020000);

    // (barriers: nch + 1 in either loop, as in gemm_bf16x3_pc_kernel)
    int fired = 0;
    v16f acc[2][2];
    if (producer) {
        v4f ra[PC_AHEAD][2], rb[PC_AHEAD][2];
        const auto load_both = [&](int c, v4f (&xa)[2], v4f (&xb)[2]) {
            if (MODE == LOAD_K_CONTIG) {
                load_kcontig_buffer<K4>(rsrc_a, static_cast<uint32_t>(p.a_rs) * 4u, m0, p.M, c * BK, p.K, ptid, xa);
                load_kcontig_buffer<K4>(rsrc_b, static_cast<uint32_t>(p.b_rs) * 4u, n0, p.N, c * BK, p.K, ptid, xb);
            } else {
                load_rows8_buffer(rsrc_a, static_cast<uint32_t>(p.a_ks) * 4u, m0, p.M, c * BK, ptid, xa);
                load_rows8_buffer(rsrc_b, static_cast<uint32_t>(p.b_ks) * 4u, n0, p.N, c * BK, ptid, xb);
            }
        };
#pragma unroll
        for (int d = 0; d < PC_AHEAD; ++d)
            if (d < nch) load_both(c_begin + d, ra[d], rb[d]);
        SplitGuard guard;
        for (int cg = 0; cg < nch; cg += PC_AHEAD) {
#pragma unroll
            for (int d = 0; d < PC_AHEAD; ++d) {
                const int c = cg + d;
                if (c >= nch) break;                    // uniform
                uint8_t* half = lds_ab[c & 1];
                split_store<MODE>(half, ptid, ra[d], guard);
                split_store<MODE>(half + STAGE, ptid, rb[d], guard);
                if (c + PC_AHEAD < nch) load_both(c_begin + c + PC_AHEAD, ra[d], rb[d]);
                __syncthreads();
            }
        }
        __syncthreads();
        fired = guard.fired() ? 1 : 0;
    } else {
#pragma unroll
    for (int ti = 0; ti < 2; ++ti)
#pragma unroll
        for (int tj = 0; tj < 2; ++tj)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[ti][tj][r] = 0.0f;
    const int frag_a = (wm + j) * SPLIT_PITCH + hh * 16;
    const int frag_b = STAGE + (wn + j) * SPLIT_PITCH + hh * 16;
    __syncthreads();                                    // chunk 0 is in LDS
    for (int c = 0; c < nch; ++c) {
        const uint8_t* half = lds_ab[c & 1];
        v8bf fa[2][3], fb[2][3];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int s3 = 0; s3 < 3; ++s3) {
                fa[t][s3] = *reinterpret_cast<const v8bf*>(half + frag_a + s3 * SPLIT_PLANE + t * 32 * SPLIT_PITCH);
                fb[t][s3] = *reinterpret_cast<const v8bf*>(half + frag_b + s3 * SPLIT_PLANE + t * 32 * SPLIT_PITCH);
            }
#pragma unroll
        for (int q = 0; q < 6; ++q)
#pragma unroll
            for (int ti = 0; ti < 2; ++ti)
#pragma unroll
                for (int tj = 0; tj < 2; ++tj)
                    acc[ti][tj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[ti][SPLIT_TERMS[q][0]], fb[tj][SPLIT_TERMS[q][1]], acc[ti][tj], 0, 0, 0);
        __syncthreads();                                // chunk c has been read; chunk c + 1 is in LDS
    }
    }
    const bool again = __syncthreads_or(fired) != 0;    // an operand of this tile and slice that the split could not carry
    if (producer) return;
    // raw sums of this slice (NaN for a tile to be computed again): the padded workspace takes every row and column of the tile
    float* dst = partial + (static_cast<size_t>(slice) * ma_pad + m0 + wm + 4 * hh) * nb_pad + n0 + wn + j;
    const float nan = __builtin_nanf("");
#pragma unroll
    for (int ti = 0; ti < 2; ++ti)
#pragma unroll
        for (int tj = 0; tj < 2; ++tj)
#pragma unroll
            for (int r = 0; r < 16; ++r) dst[static_cast<size_t>(ti * 32 + 8 * (r >> 2) + (r & 3)) * nb_pad + tj * 32] = again ? nan : acc[ti][tj][r];
}

// The same again for contractions with one NARROW side: at most 32 rows of A (SIDE_M: the second contraction of the
// attention chain, out_prod_tt_hip with the head dimension for its rows) or of B (SIDE_N: a LinearLayer with up to 32
// output features -- the bias projections onto the heads, the 256 -> 16 projections of the outer-product-mean).  A 128 x
// 128 tile is three quarters padding there: matrix work, split and LDS traffic for rows that do not exist.  Here the
// tile is 128 along the long side and 32 along the narrow one; each of the four contracting waves takes 32 rows of the
// long operand against the one fragment of the narrow operand, six MFMAs per 16-k chunk; of the loading waves all
// four split the long operand and two of them (one, with contiguous rows) the narrow one.  Operands contiguous in k
// (MODE LOAD_K_CONTIG) or in their rows (LOAD_ROW_CONTIG: the backward of the attention logits, out_prod(grad,
// mat_transpose(Q)), 256 x 32 per plane under K = 256), buffer addressing, same products in the same order as the other
// forms: same bits.
constexpr int SIDE_M = 1, SIDE_N = 2;
template <int MODE, int SIDE, bool STREAM_C, bool K4>
__global__ __launch_bounds__(512) void gemm_bf16x3_pc_narrow_kernel(const GemmParams p) {
    static_assert(SIDE == SIDE_M || SIDE == SIDE_N, "which operand is the narrow one");
    static_assert(MODE == LOAD_ROW_CONTIG || MODE == LOAD_K_CONTIG, "buffer addressing");
    constexpr int LONG_STAGE = 3 * SPLIT_PLANE;                  // three planes of 128 rows
    constexpr int NARROW_PLANE = 32 * SPLIT_PITCH;
    constexpr int STAGE = LONG_STAGE + 3 * NARROW_PLANE;
    __shared__ __attribute__((aligned(16))) uint8_t lds_ab[2][STAGE];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 31, hh = lane >> 5;
    const bool producer = wave >= 4;
    const int ptid = tid & 255;
    const int cw = wave & 3;

    // the tile list runs along the long side only (the launcher sets tiles_m or tiles_n to 1 for the narrow side)
    int plane, m0, n0;
    tile_of_group(p, plane, m0, n0);
    const int p2 = plane % p.np2, p3 = plane / p.np2;
    const float* A = p.A + p2 * p.a_p2 + p3 * p.a_p3;
    const float* B = p.B + (p2 / p.b_div2) * p.b_p2 + (p3 / p.b_div3) * p.b_p3;
    float* C = p.C + p2 * p.c_p2 + p3 * p.c_p3;
    const int chunks = (p.K + BK - 1) / BK;

    const int64_t a_plane = MODE == LOAD_K_CONTIG ? (p.M - 1) * p.a_rs + p.K : p.K * p.a_ks;
    const int64_t b_plane = MODE == LOAD_K_CONTIG ? (p.N - 1) * p.b_rs + p.K : p.K * p.b_ks;
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(A), 0, static_cast<int>(a_plane * 4), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(B), 0, static_cast<int>(b_plane * 4), 0x00020000);
    const __amdgpu_buffer_rsrc_t& rsrc_long = SIDE == SIDE_M ? rsrc_b : rsrc_a;
    const __amdgpu_buffer_rsrc_t& rsrc_narrow = SIDE == SIDE_M ? rsrc_a : rsrc_b;
    // the step between rows (k-contiguous operands) or between k (row-contiguous ones), in bytes
    const uint32_t long_rs = static_cast<uint32_t>(MODE == LOAD_K_CONTIG ? (SIDE == SIDE_M ? p.b_rs : p.a_rs) : (SIDE == SIDE_M ? p.b_ks : p.a_ks)) * 4u;
    const uint32_t narrow_rs = static_cast<uint32_t>(MODE == LOAD_K_CONTIG ? (SIDE == SIDE_M ? p.a_rs : p.b_rs) : (SIDE == SIDE_M ? p.a_ks : p.b_ks)) * 4u;
    const int long_row0 = SIDE == SIDE_M ? n0 : m0, long_rows = SIDE == SIDE_M ? p.N : p.M;
    const int narrow_rows = SIDE == SIDE_M ? p.M : p.N;

    // (barriers: chunks + 1 in either loop, as in gemm_bf16x3_pc_kernel)
    int fired = 0;
    if (producer) {
        v4f rl[PC_AHEAD][2];                            // the long operand: two row pieces per thread (one row, eight k, with contiguous rows)
        v4f rn[PC_AHEAD][2];                            // the narrow one: one piece per thread of the first two loading waves (eight k per thread of the first)
        const bool has_narrow = MODE == LOAD_K_CONTIG ? wave < 6 : wave < 5;     // rows ptid / 4 < 32; row ptid % 32, k half ptid / 32 of 64 threads
        const auto load_both = [&](int c, v4f (&xl)[2], v4f (&xn)[2]) {
            if (MODE == LOAD_K_CONTIG) {
                load_kcontig_buffer<K4>(rsrc_long, long_rs, long_row0, long_rows, c * BK, p.K, ptid, xl);
                if (has_narrow) {
                    const int k = c * BK + (ptid & 3) * 4;
                    const int row = ptid >> 2;
                    const uint32_t at = row < narrow_rows ? static_cast<uint32_t>(row) * narrow_rs + static_cast<uint32_t>(k) * 4u : OUTSIDE;
                    if (K4) {
                        xn[0] = __builtin_bit_cast(v4f, __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_narrow, k < p.K ? at : OUTSIDE, 0, 0)));
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            xn[0][e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc_narrow, k + e < p.K ? at + 4u * e : OUTSIDE, 0, 0));
                    }
                }
            } else {
                load_rows8_buffer(rsrc_long, long_rs, long_row0, long_rows, c * BK, ptid, xl);
                if (has_narrow) {
                    const int row = ptid & 31;
                    const uint32_t lane_off = row < narrow_rows ? static_cast<uint32_t>(row) * 4u : OUTSIDE;
                    const uint32_t kb = static_cast<uint32_t>(c * BK + (ptid >> 5) * 8);
#pragma unroll
                    for (int e = 0; e < 8; ++e)     // (k past the end: outside the plane, whose size is K steps)
                        xn[e >> 2][e & 3] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc_narrow, lane_off + (kb + e) * narrow_rs, 0, 0));
                }
            }
        };
#pragma unroll
        for (int d = 0; d < PC_AHEAD; ++d)
            if (d < chunks) load_both(d, rl[d], rn[d]);
        SplitGuard guard;
        for (int cg = 0; cg < chunks; cg += PC_AHEAD) {
#pragma unroll
            for (int d = 0; d < PC_AHEAD; ++d) {
                const int c = cg + d;
                if (c >= chunks) break;                 // uniform
                uint8_t* half = lds_ab[c & 1];
                split_store<MODE>(half, ptid, rl[d], guard);
                if (has_narrow) {
                    if (MODE == LOAD_K_CONTIG) {
                        uint2 parts[3];
                        split4(rn[d][0], parts, guard);
                        uint8_t* dst = half + LONG_STAGE + (ptid >> 2) * SPLIT_PITCH + (ptid & 3) * 8;
#pragma unroll
                        for (int s3 = 0; s3 < 3; ++s3) *reinterpret_cast<uint2*>(dst + s3 * NARROW_PLANE) = parts[s3];
                    } else {
                        uint2 lo[3], hi[3];
                        split4(rn[d][0], lo, guard);
                        split4(rn[d][1], hi, guard);
                        uint8_t* dst = half + LONG_STAGE + (ptid & 31) * SPLIT_PITCH + (ptid >> 5) * 16;
#pragma unroll
                        for (int s3 = 0; s3 < 3; ++s3) *reinterpret_cast<uint4*>(dst + s3 * NARROW_PLANE) = uint4{lo[s3].x, lo[s3].y, hi[s3].x, hi[s3].y};
                    }
                }
                if (c + PC_AHEAD < chunks) load_both(c + PC_AHEAD, rl[d], rn[d]);
                __syncthreads();
            }
        }
        __syncthreads();
        fired = guard.fired() ? 1 : 0;
    }

    v16f acc;
    if (!producer) {
        {
            const int n = SIDE == SIDE_M ? n0 + cw * 32 + j : j;
            const float b0 = (p.bias && n < p.N) ? p.bias[n] : 0.0f;
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[r] = b0;
        }
        const int frag_long = (cw * 32 + j) * SPLIT_PITCH + hh * 16;
        const int frag_narrow = LONG_STAGE + j * SPLIT_PITCH + hh * 16;
        __syncthreads();                                // chunk 0 is in LDS
        for (int c = 0; c < chunks; ++c) {
            const uint8_t* half = lds_ab[c & 1];
            v8bf fl[3], fn[3];
#pragma unroll
            for (int s3 = 0; s3 < 3; ++s3) {
                fl[s3] = *reinterpret_cast<const v8bf*>(half + frag_long + s3 * SPLIT_PLANE);
                fn[s3] = *reinterpret_cast<const v8bf*>(half + frag_narrow + s3 * NARROW_PLANE);
            }
#pragma unroll
            for (int q = 0; q < 6; ++q) {
                // (part of a, part of b): a is the narrow operand with SIDE_M, the long one with SIDE_N
                const v8bf& fa = SIDE == SIDE_M ? fn[SPLIT_TERMS[q][0]] : fl[SPLIT_TERMS[q][0]];
                const v8bf& fb = SIDE == SIDE_M ? fl[SPLIT_TERMS[q][1]] : fn[SPLIT_TERMS[q][1]];
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb, acc, 0, 0, 0);
            }
            __syncthreads();
        }
    }

    if (__syncthreads_or(fired)) {
        // the whole tile again, the reference's way: 128 along the long side, the narrow side in full
        if (tid < 256) plain_tile(p, A, B, C, SIDE == SIDE_M ? 0 : m0, SIDE == SIDE_M ? n0 : 0, SIDE == SIDE_M ? 32 : BM, SIDE == SIDE_M ? BN : 32, tid);
        return;
    }
    if (!producer) {
        const __amdgpu_buffer_rsrc_t rsrc_c = __builtin_amdgcn_make_buffer_rsrc(C, 0, static_cast<int>(p.M * p.c_mi * 4), 0x00020000);
        const uint32_t ld_bytes = static_cast<uint32_t>(p.c_mi) * 4u;
        const int m_base = SIDE == SIDE_M ? 0 : m0 + cw * 32;
        const int n = SIDE == SIDE_M ? n0 + cw * 32 + j : j;
        const uint32_t first = static_cast<uint32_t>(m_base + 4 * hh);
        // rows past the matrix fall outside the plane by themselves (offset >= M * ld bytes)
        const uint32_t base = n < p.N ? first * ld_bytes + static_cast<uint32_t>(n) * 4u : OUTSIDE;
        const bool scale = p.alpha != 1.0f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            float v = acc[r];
            if (scale) v *= p.alpha;
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), rsrc_c, base + (8 * (r >> 2) + (r & 3)) * ld_bytes, 0, STREAM_C ? 3 : 0);
        }
    }
}

// A long, tall operand with compound indices against a small one (the outer-product-mean backward: the gradient
// tensor [d1][d2][i][j], 12288 x 12288 at the configured size, against 256 columns).  Splitting the tall operand ahead,
// as gemm_planes_kernel wants it, reads it element by element and moves 2.5 times its bytes before the matrix work
// starts -- as long as the matrix work itself.  Here only the SMALL operand is split ahead (split_operand_kernel, any
// strides); the contracting waves read its fragments straight from memory (L2), HS_AHEAD chunks ahead, one wave per 32
// columns, and the loading waves split the tall operand as in gemm_bf16x3_pc_kernel, from loads that follow its runs:
// the compound index is resolved once per lane for the rows (a byte offset) and by a scalar cursor for the chunks
// (run number and place within the run of a chunk's first k), so a load is one add.  HS_KRUN: the contraction index
// runs along memory (sixteen bytes per load); HS_RRUN: the row index does (eight loads, each contiguous across the
// lanes).  GEN: runs of any length (a pair tensor of 103 residues): a chunk may then pass from one run into the next and
// end behind the last one, so every element takes its own load, whose offset is picked between the two runs' bases.
// The K loop is cut into slices (tile numbering: the slice is the plane; one slice is allowed): raw sums go to
// partial[slice][m][n] for reduce_slices_kernel, which adds them in slice order, applies bias, factor and the output's
// addressing, and computes the rows and columns flagged here (fired_a, one per 32 rows) or by the small operand's split
// (fired_b) the reference's way.
constexpr int HS_KRUN = 0, HS_RRUN = 1;
constexpr int HS_AHEAD = 2;
template <int AMODE, bool GEN>
__global__ __launch_bounds__(512, 2) void gemm_bf16x3_half_split_kernel(const GemmParams p, const uint8_t* __restrict__ wb, int nb_pad, int chunks,
                                                                        int slice_chunks, float* __restrict__ partial, int ma_pad,
                                                                        int* __restrict__ fired_a, uint32_t a_span_bytes) {
    constexpr int STAGE = 3 * SPLIT_PLANE;
    constexpr int SMODE = AMODE == HS_KRUN ? LOAD_K_CONTIG : LOAD_ROW_CONTIG;     // the thread-to-element mapping of the split
    __shared__ __attribute__((aligned(16))) uint8_t lds_a[2][STAGE];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 31, hh = lane >> 5;
    const bool producer = wave >= 4;
    const int ptid = tid & 255;
    const int wn = (wave & 3) * 32;

    int slice, m0, n0;
    tile_of_group(p, slice, m0, n0);
    const int c_begin = slice * slice_chunks;
    const int c_end = c_begin + slice_chunks < chunks ? c_begin + slice_chunks : chunks;
    const int nch = c_end - c_begin;
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.A), 0, static_cast<int>(a_span_bytes), 0x00020000);

    // (barriers: nch + 1 in either loop, as in gemm_bf16x3_pc_kernel)
    if (producer) {
        // byte offsets of this lane's rows (and, HS_KRUN, of its four k within a chunk); 2^31 for rows past the matrix
        uint32_t roff[2];
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            const int row = AMODE == HS_KRUN ? m0 + (ptid >> 2) + it * 64 : m0 + (ptid & 127);
            const int64_t el = static_cast<int64_t>(row / p.a_lm) * p.a_mo + static_cast<int64_t>(row % p.a_lm) * p.a_mi;
            roff[it] = row < p.M ? static_cast<uint32_t>(el) * 4u + (AMODE == HS_KRUN ? (ptid & 3) * 16u : 0u) : OUTSIDE;
        }
        // the chunk the next load is for: run number and place within the run of its first k
        int kd = (c_begin * BK) / p.a_lk, kr = (c_begin * BK) % p.a_lk;
        const int nruns = p.K / p.a_lk;
        const int oct = __builtin_amdgcn_readfirstlane(ptid >> 7) * 8;
        const auto load = [&](v4f (&x)[2]) {
            if (!GEN) {                                 // runs of whole chunks
                if (AMODE == HS_KRUN) {
                    const uint32_t koff = static_cast<uint32_t>(static_cast<int64_t>(kd) * p.a_ko + kr) * 4u;
#pragma unroll
                    for (int it = 0; it < 2; ++it) x[it] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, roff[it] + koff, 0, 0));
                } else {
#pragma unroll
                    for (int c = 0; c < 8; ++c) {
                        const uint32_t koff = static_cast<uint32_t>(static_cast<int64_t>(kd) * p.a_ko + static_cast<int64_t>(kr + oct + c) * p.a_ki) * 4u;
                        x[c >> 2][c & 3] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc_a, roff[0] + koff, 0, 0));
                    }
                }
            } else {
                // element u places behind the chunk's first k lies in this run while kr + u < run length, else in the next
                // one (a run is at least a chunk long: the launcher's rule); a run behind the last one is outside: 2^30,
                // which with the operand's span (at most 2^30 bytes in this form) and with a row's 2^31 stays outside
                constexpr uint32_t NO_RUN = 0x40000000u;
                const uint32_t here = kd < nruns ? static_cast<uint32_t>(static_cast<int64_t>(kd) * p.a_ko + static_cast<int64_t>(kr) * p.a_ki) * 4u : NO_RUN;
                const uint32_t next = kd + 1 < nruns ? static_cast<uint32_t>(static_cast<int64_t>(kd + 1) * p.a_ko + static_cast<int64_t>(kr - p.a_lk) * p.a_ki) * 4u : NO_RUN;
                const int left = p.a_lk - kr;             // elements of the chunk that lie in this run
                if (AMODE == HS_KRUN) {
                    const int u0 = (ptid & 3) * 4;
#pragma unroll
                    for (int it = 0; it < 2; ++it)
#pragma unroll
                        for (int e = 0; e < 4; ++e) {       // (k step 1: the place within the chunk is part of roff)
                            const uint32_t base = u0 + e < left ? here : next;
                            x[it][e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc_a, roff[it] + base + 4u * e, 0, 0));
                        }
                } else {
                    const uint32_t step = static_cast<uint32_t>(p.a_ki) * 4u;
#pragma unroll
                    for (int c = 0; c < 8; ++c) {
                        const uint32_t koff = (oct + c < left ? here : next) + static_cast<uint32_t>(oct + c) * step;
                        x[c >> 2][c & 3] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc_a, roff[0] + koff, 0, 0));
                    }
                }
            }
            kr += BK;
            if (kr >= p.a_lk) { kr -= p.a_lk; ++kd; }
        };
        v4f ra[PC_AHEAD][2];
#pragma unroll
        for (int d = 0; d < PC_AHEAD; ++d)
            if (d < nch) load(ra[d]);
        SplitGuard guard;
        for (int cg = 0; cg < nch; cg += PC_AHEAD) {
#pragma unroll
            for (int d = 0; d < PC_AHEAD; ++d) {
                const int c = cg + d;
                if (c >= nch) break;                    // uniform
                split_store<SMODE>(lds_a[c & 1], ptid, ra[d], guard);
                if (c + PC_AHEAD < nch) load(ra[d]);
                __syncthreads();
            }
        }
        __syncthreads();
        if (guard.fired()) {                            // (every writer writes the same value)
            if (AMODE == HS_KRUN) { fired_a[(m0 + (ptid >> 2)) >> 5] = 1; fired_a[(m0 + (ptid >> 2) + 64) >> 5] = 1; }
            else fired_a[(m0 + (ptid & 127)) >> 5] = 1;
        }
        return;
    }

    v16f acc[4];
    {
#pragma unroll
        for (int ti = 0; ti < 4; ++ti)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[ti][r] = 0.0f;
        const size_t b_chunk = static_cast<size_t>(nb_pad) * 32, b_part = b_chunk * chunks;
        const uint8_t* bfrag = wb + static_cast<size_t>(n0 + wn) * 32 + lane * 16 + c_begin * b_chunk;
        const int frag_a = j * SPLIT_PITCH + hh * 16;
        v8bf fb[HS_AHEAD + 1][3];                       // sets that take turns by name (the loop body is written out three times)
        const auto load_fb = [&](v8bf (&f)[3], int c) {
#pragma unroll
            for (int s3 = 0; s3 < 3; ++s3) f[s3] = *reinterpret_cast<const v8bf*>(bfrag + s3 * b_part + c * b_chunk);
        };
#pragma unroll
        for (int d = 0; d < HS_AHEAD; ++d)
            if (d < nch) load_fb(fb[d], d);
        __syncthreads();                                // chunk 0 of the tall operand is in LDS
        for (int cg = 0; cg < nch; cg += HS_AHEAD + 1) {
#pragma unroll
            for (int u = 0; u < HS_AHEAD + 1; ++u) {
                const int c = cg + u;
                if (c >= nch) break;                    // uniform
                if (c + HS_AHEAD < nch) load_fb(fb[(u + HS_AHEAD) % (HS_AHEAD + 1)], c + HS_AHEAD);
                const uint8_t* half = lds_a[c & 1];
#pragma unroll
                for (int ti = 0; ti < 4; ++ti) {
                    v8bf fa[3];
#pragma unroll
                    for (int s3 = 0; s3 < 3; ++s3) fa[s3] = *reinterpret_cast<const v8bf*>(half + frag_a + s3 * SPLIT_PLANE + ti * 32 * SPLIT_PITCH);
#pragma unroll
                    for (int q = 0; q < 6; ++q)
                        acc[ti] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[SPLIT_TERMS[q][0]], fb[u][SPLIT_TERMS[q][1]], acc[ti], 0, 0, 0);
                }
                __syncthreads();
            }
        }
    }

    // raw sums of this slice: the padded workspace takes every row and column of the tile
    float* dst = partial + (static_cast<size_t>(slice) * ma_pad + m0 + 4 * hh) * nb_pad + n0 + wn + j;
#pragma unroll
    for (int ti = 0; ti < 4; ++ti)
#pragma unroll
        for (int r = 0; r < 16; ++r) dst[static_cast<size_t>(ti * 32 + 8 * (r >> 2) + (r & 3)) * nb_pad] = acc[ti][r];
}

// ------------------------------------------------------------------------------------------
// Batched contractions with a short K (at most 32: the attention logits, K = head dimension) on operands whose
// rows are contiguous, into dense output planes.  Per output tile there are two 16-k chunks of matrix work and
// TM x TM x 4 bytes to write, so a work-group that does one tile is a chain load -> split -> MFMA -> store
// whose stages wait for each other, and the kernel above ran at 0.45 (pair shape) and 0.75 (MSA shape) of what
// its bytes alone take.  This form is persistent and staged the other way round:
//
//   * two work-groups per CU walk the tile list; the tiles of one XCD are consecutive ones, so the two or
//     four tiles that share an operand panel meet in one L2;
//   * the whole K of a tile is loaded at once (every lane: one row, eight k, per operand and 16-k chunk), and
//     the loads of tile i + 1 are issued before the matrix work of tile i; they are older than tile i's stores,
//     so waiting for them at the top of the next iteration does not wait for those stores;
//   * both chunks are split into LDS together: two barriers per tile, no load inside the matrix work;
//   * addresses through one buffer resource per plane (rows and columns outside the matrix: zero on the way
//     in, dropped on the way out).
//
// Arithmetic and order of the sums are those of gemm_bf16x3_kernel: same bits.
//
// C_FORM says how a tile leaves: C_ORDINARY / C_STREAM store the accumulator registers as they lie (a store
// instruction writes 32 consecutive floats of two rows: whole 128-byte lines only when the rows are), C_FLAT is for
// dense planes whose rows are NOT whole lines and a tile that spans all columns (N <= TM): the rows of the tile are then
// one contiguous range of memory, which goes through LDS (free once the matrix work is done) and leaves as whole,
// aligned lines by streaming stores -- rows that end anywhere inside a line no longer leave partly written lines
// behind in L2 -- except for the first and last line of the range, which it shares with its neighbours.  C_ROWS is
// for rows of whole lines that are longer than the tile is wide: the tile goes through LDS as well and leaves
// sixteen bytes per lane, a store instruction writing two 512-byte runs instead of two lines.
constexpr int C_ORDINARY = 0, C_STREAM = 1, C_FLAT = 2, C_ROWS = 3;
template <int TM, int C_FORM>
__global__ __launch_bounds__(256, 2) void gemm_bf16x3_shortk_kernel(const GemmParams p, int total_tiles, uint32_t launch_mark) {
    static_assert(TM == 64 || TM == 128, "tile side");
    constexpr int WT = TM / 2;                        // a wave's square of the tile
    constexpr int NT = WT / 32;                       // 32 x 32 accumulator tiles per side of it
    constexpr int CHUNK_PLANE = TM * SPLIT_PITCH;     // one bf16 plane of one 16-k chunk of one operand
    constexpr int OPERAND = 2 * 3 * CHUNK_PLANE;      // [chunk][plane][row][48 bytes]
    constexpr int LOADS = TM == 128 ? 2 : 1;          // 16-k chunks a thread loads separately (at 64 rows one pass covers K = 32)
    static_assert(2 * OPERAND >= (TM * TM + 32) * 4, "a whole tile of C, shifted by up to a line, fits the operands' LDS");
    __shared__ __attribute__((aligned(128))) uint8_t lds_ab[2 * OPERAND];
    // "A SplitGuard fired for tile t": a thread whose guard fires writes a mark into the word of t's turn, and after
    // the barrier everybody compares.  LDS keeps what earlier kernels left there -- this kernel's own marks
    // (work-groups land on the same CUs launch after launch) and whatever other kernels kept at these addresses, which
    // may well look like a tile number: a word taken for a mark sends its tile down the plain path (right results, the
    // other path's bits, fifteen times the time).  So a mark is a word that nothing else writes -- a scrambled count
    // of the host's launches (the kernel's last argument) with the tile's number folded in --, and a work-group that
    // saw one clears the words before it ends (a captured graph replays the same launch number).  What is left is one
    // chance in 2^32 per tile that leftover data is taken for a mark: that tile then has the other path's bits, once.
    // (Clearing the words when the kernel starts takes a barrier in front of the first split, or a mark written behind
    // the split's barrier: 0.2 to 0.35 us per launch either way; a second word to compare, about as much.)
    __shared__ uint32_t lds_guard[2];
    uint8_t* const lds_a = lds_ab;
    uint8_t* const lds_b = lds_ab + OPERAND;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 31, hh = lane >> 5;
    const int wm = (wave >> 1) * WT, wn = (wave & 1) * WT;
    const int tiles_m = (p.M + TM - 1) / TM, tiles_n = (p.N + TM - 1) / TM;
    const int per_plane = tiles_m * tiles_n;

    // this work-group's tiles: the list is cut into eight consecutive parts, one per XCD (work-group ids go
    // round the XCDs), and the work-groups of an XCD take the tiles of its part in turn
    constexpr int XCDS = 8;
    const int groups = static_cast<int>(gridDim.x) / XCDS;                 // work-groups per XCD (the grid is a multiple of 8)
    const int xcd = static_cast<int>(blockIdx.x) % XCDS, slot = static_cast<int>(blockIdx.x) / XCDS;
    const int part = (total_tiles + XCDS - 1) / XCDS;
    const int part_begin = xcd * part;
    const int part_end = part_begin + part < total_tiles ? part_begin + part : total_tiles;

    // thread -> (row of the tile, octet of k) for the loads and the split
    const int lrow = TM == 128 ? (tid & 127) : (tid & 63);
    const int loct = TM == 128 ? (tid >> 7) : (tid >> 6);                  // uniform within a wave
    v4f ra[LOADS][2], rb[LOADS][2];

    struct Tile { const float* A; const float* B; float* C; int m0, n0; };
    const auto tile_at = [&](int t) {
        const int plane = t / per_plane;
        const int r = t - plane * per_plane;
        const int p2 = plane % p.np2, p3 = plane / p.np2;
        Tile tl;
        tl.A = p.A + p2 * p.a_p2 + p3 * p.a_p3;
        tl.B = p.B + (p2 / p.b_div2) * p.b_p2 + (p3 / p.b_div3) * p.b_p3;
        tl.C = p.C + p2 * p.c_p2 + p3 * p.c_p3;
        tl.m0 = (r / tiles_n) * TM;
        tl.n0 = (r % tiles_n) * TM;
        return tl;
    };
    const uint32_t a_ks = static_cast<uint32_t>(p.a_ks) * 4u, b_ks = static_cast<uint32_t>(p.b_ks) * 4u;
    const int a_bytes = static_cast<int>(p.K * p.a_ks * 4), b_bytes = static_cast<int>(p.K * p.b_ks * 4);
    const auto load_tile_regs = [&](const Tile& tl) {
        const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(tl.A), 0, a_bytes, 0x00020000);
        const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(tl.B), 0, b_bytes, 0x00020000);
        const uint32_t off_a = tl.m0 + lrow < p.M ? static_cast<uint32_t>(tl.m0 + lrow) * 4u : OUTSIDE;
        const uint32_t off_b = tl.n0 + lrow < p.N ? static_cast<uint32_t>(tl.n0 + lrow) * 4u : OUTSIDE;
#pragma unroll
        for (int l = 0; l < LOADS; ++l) {
            const uint32_t kb = static_cast<uint32_t>((TM == 128 ? l * 16 : 0) + __builtin_amdgcn_readfirstlane(loct) * 8);
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                // k >= K lies behind the end of the plane: zero
                ra[l][c >> 2][c & 3] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc_a, off_a + (kb + c) * a_ks, 0, 0));
                rb[l][c >> 2][c & 3] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc_b, off_b + (kb + c) * b_ks, 0, 0));
            }
        }
    };
    // a lane's share goes to the three planes of its chunk: row lrow, bytes 16 * (octet % 2) of the row's 32
    const auto split_to_lds = [&](uint32_t* fired, uint32_t mark) {
        SplitGuard guard;
#pragma unroll
        for (int l = 0; l < LOADS; ++l) {
            const int oct = (TM == 128 ? 2 * l : 0) + loct;                 // octet of k, 0..3
            const int at = (oct >> 1) * 3 * CHUNK_PLANE + lrow * SPLIT_PITCH + (oct & 1) * 16;
            uint2 lo[3], hi[3];
            split4(ra[l][0], lo, guard);
            split4(ra[l][1], hi, guard);
#pragma unroll
            for (int q = 0; q < 3; ++q) *reinterpret_cast<uint4*>(lds_a + at + q * CHUNK_PLANE) = uint4{lo[q].x, lo[q].y, hi[q].x, hi[q].y};
            split4(rb[l][0], lo, guard);
            split4(rb[l][1], hi, guard);
#pragma unroll
            for (int q = 0; q < 3; ++q) *reinterpret_cast<uint4*>(lds_b + at + q * CHUNK_PLANE) = uint4{lo[q].x, lo[q].y, hi[q].x, hi[q].y};
        }
        if (guard.fired()) *fired = mark;               // (every writer writes the same value)
    };

    int t = part_begin + slot;
    if (t >= part_end) return;                          // whole work-group: no barrier is left behind
    int turn = 0;
    uint64_t fired_its = 0;                             // the tiles of this loop for which a SplitGuard fired (see below)
    int it = 0;
    Tile cur = tile_at(t);
    load_tile_regs(cur);
    const uint8_t* frag_a = lds_a + (wm + j) * SPLIT_PITCH + hh * 16;
    const uint8_t* frag_b = lds_b + (wn + j) * SPLIT_PITCH + hh * 16;
    const bool scale = p.alpha != 1.0f;
    const uint32_t ld_bytes = static_cast<uint32_t>(p.c_mi) * 4u;
    const int c_bytes = static_cast<int>(p.M * p.c_mi * 4);

    while (true) {
        // An operand of this tile that the split could not carry: the tile is stored as the matrix pipe leaves it all the
        // same, the loop only notes which of its tiles that was (a mark in the LDS word of the tile's turn, read behind
        // the matrix work), and the work-group writes those tiles again, the reference's way, when the loop has ended.
        // That keeps the test and the other path's code out of the chain load -> split -> MFMA -> store that a
        // work-group with one tile consists of (decided ahead of the matrix work it cost half a microsecond per
        // launch; with the other path inline behind the stores, a third).
        uint32_t* const mark_word = &lds_guard[turn];
        const uint32_t mark = launch_mark ^ static_cast<uint32_t>(t + 1);
        split_to_lds(mark_word, mark);
        __syncthreads();
        turn ^= 1;
        const int t_next = t + groups;
        const bool more = t_next < part_end;
        Tile nxt = cur;
        if (more) {
            nxt = tile_at(t_next);
            load_tile_regs(nxt);
        }
        v16f acc[NT][NT];
#pragma unroll
        for (int ti = 0; ti < NT; ++ti)
#pragma unroll
            for (int tj = 0; tj < NT; ++tj)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[ti][tj][r] = 0.0f;
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            v8bf fa[NT][3], fb[NT][3];
#pragma unroll
            for (int ti = 0; ti < NT; ++ti)
#pragma unroll
                for (int q = 0; q < 3; ++q) {
                    fa[ti][q] = *reinterpret_cast<const v8bf*>(frag_a + (c * 3 + q) * CHUNK_PLANE + ti * 32 * SPLIT_PITCH);
                    fb[ti][q] = *reinterpret_cast<const v8bf*>(frag_b + (c * 3 + q) * CHUNK_PLANE + ti * 32 * SPLIT_PITCH);
                }
#pragma unroll
            for (int q = 0; q < 6; ++q)
#pragma unroll
                for (int ti = 0; ti < NT; ++ti)
#pragma unroll
                    for (int tj = 0; tj < NT; ++tj)
                        acc[ti][tj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[ti][SPLIT_TERMS[q][0]], fb[tj][SPLIT_TERMS[q][1]], acc[ti][tj], 0, 0, 0);
        }
        __syncthreads();                                // the planes may be overwritten
        if (__builtin_amdgcn_readfirstlane(*mark_word) == mark) fired_its |= 1ull << (it < 63 ? it : 63);   // uniform over the work-group
        ++it;
        // ---- stores of this tile: younger than the next tile's loads
        if (C_FORM == C_FLAT) {
            // The tile's rows m0 .. m0 + rows - 1 are the floats [0, total) behind row_base.  In LDS float e of that
            // range sits at shift + e, shift = floats between the start of row_base's 128-byte line and row_base: a
            // 16-byte piece of LDS then is an aligned 16-byte piece of memory.
            float* const stage = reinterpret_cast<float*>(lds_ab);
            float* const row_base = cur.C + static_cast<int64_t>(cur.m0) * p.N;
            const int shift = static_cast<int>((reinterpret_cast<uintptr_t>(row_base) & 127) >> 2);
            const int rows = p.M - cur.m0 < TM ? static_cast<int>(p.M) - cur.m0 : TM;
            const int total = rows * static_cast<int>(p.N);
#pragma unroll
            for (int ti = 0; ti < NT; ++ti)
#pragma unroll
                for (int tj = 0; tj < NT; ++tj) {
                    const int n = wn + tj * 32 + j;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int row = wm + ti * 32 + 4 * hh + 8 * (r >> 2) + (r & 3);
                        float v = acc[ti][tj][r];
                        if (scale) v *= p.alpha;
                        // (rows past the matrix land behind the range that is stored: no test)
                        if (n < p.N) stage[shift + row * static_cast<int>(p.N) + n] = v;
                    }
                }
            __syncthreads();
            float* const line_base = row_base - shift;            // 128-byte aligned
            const int end = shift + total;
            const int whole_begin = shift ? 32 : 0;               // floats of LDS that lie in lines this tile owns alone
            const int whole_end = end & ~31;
            // every piece is read before the first is stored: one LDS round trip per tile, not one per piece
            constexpr int PIECES = (TM * TM + 32 + 1023) / 1024;
            static_assert(PIECES * 1024 * 4 <= 2 * OPERAND, "the pieces past the tile still lie in the operands' LDS");
            v4f piece[PIECES];
#pragma unroll
            for (int i = 0; i < PIECES; ++i) piece[i] = *reinterpret_cast<const v4f*>(stage + (tid + 256 * i) * 4);
#pragma unroll
            for (int i = 0; i < PIECES; ++i) {
                const int q = (tid + 256 * i) * 4;
                if (q >= whole_begin && q + 4 <= whole_end) {
                    __builtin_nontemporal_store(piece[i], reinterpret_cast<v4f*>(line_base + q));
                } else if (q + 4 > shift && q < end) {
#pragma unroll
                    for (int c = 0; c < 4; ++c)
                        if (q + c >= shift && q + c < end) line_base[q + c] = piece[i][c];
                }
            }
            if (!more) break;
            __syncthreads();                            // the staged tile has been read: the next split may overwrite it
            t = t_next;
            cur = nxt;
            continue;
        }
        if (C_FORM == C_ROWS) {
            // rows of whole lines: the tile goes to LDS as [row][TM] and leaves sixteen bytes per lane
            float* const stage = reinterpret_cast<float*>(lds_ab);
#pragma unroll
            for (int ti = 0; ti < NT; ++ti)
#pragma unroll
                for (int tj = 0; tj < NT; ++tj)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int row = wm + ti * 32 + 4 * hh + 8 * (r >> 2) + (r & 3);
                        float v = acc[ti][tj][r];
                        if (scale) v *= p.alpha;
                        stage[row * TM + wn + tj * 32 + j] = v;
                    }
            __syncthreads();
            constexpr int PIECES = TM * TM / 1024;
            v4f piece[PIECES];
#pragma unroll
            for (int i = 0; i < PIECES; ++i) piece[i] = *reinterpret_cast<const v4f*>(stage + (tid + 256 * i) * 4);
            float* const tile_base = cur.C + static_cast<int64_t>(cur.m0) * p.c_mi + cur.n0;
#pragma unroll
            for (int i = 0; i < PIECES; ++i) {
                const int q = tid + 256 * i;
                const int row = q / (TM / 4), c4 = (q % (TM / 4)) * 4;
                if (cur.m0 + row < p.M && cur.n0 + c4 < p.N)
                    __builtin_nontemporal_store(piece[i], reinterpret_cast<v4f*>(tile_base + static_cast<int64_t>(row) * p.c_mi + c4));
            }
            if (!more) break;
            __syncthreads();
            t = t_next;
            cur = nxt;
            continue;
        }
        const __amdgpu_buffer_rsrc_t rsrc_c = __builtin_amdgcn_make_buffer_rsrc(cur.C, 0, c_bytes, 0x00020000);
#pragma unroll
        for (int ti = 0; ti < NT; ++ti) {
            const uint32_t first = static_cast<uint32_t>(cur.m0 + wm + ti * 32 + 4 * hh);
#pragma unroll
            for (int tj = 0; tj < NT; ++tj) {
                const int n = cur.n0 + wn + tj * 32 + j;
                const uint32_t base = n < p.N ? first * ld_bytes + static_cast<uint32_t>(n) * 4u : OUTSIDE;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    float v = acc[ti][tj][r];
                    if (scale) v *= p.alpha;
                    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), rsrc_c, base + (8 * (r >> 2) + (r & 3)) * ld_bytes, 0,
                                                          C_FORM == C_STREAM ? 3 : 0);
                }
            }
        }
        if (!more) break;
        t = t_next;
        cur = nxt;
    }
    if (fired_its != 0) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wave's stores have been acknowledged ...
        __syncthreads();                                    // ... and so have the other waves'
        if (tid < 2) lds_guard[tid] = 0;                    // (see lds_guard)
        shortk_redo_fired(fired_its, TM, tid);
    }
}

// ------------------------------------------------------------------------------------------
// F16 x F16 -> F32 (mul_mat with both operands in halves, k contiguous): the halves go to the matrix
// pipe as they are.  v_mfma_f32_32x32x16_f16 forms each product exactly (22 significant bits) and adds
// into a binary32 accumulator, which is the reference's arithmetic (src/backend/CPUKernels.cpp:763-771
// with half operands converted on load) up to the order of the additions; the bias joins the finished
// sum, as the CPU branch of the reference does.
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

// eight consecutive halves (16 bytes) of row `row`, zeros past the matrix
__device__ __forceinline__ v4i load_halves8(const uint16_t* __restrict__ base, int64_t rs, int row, int nrows, int k, int K) {
    v4i v = {0, 0, 0, 0};
    if (row < nrows && k < K) {
        const uint16_t* p = base + static_cast<int64_t>(row) * rs + k;
        if (k + 7 < K && (reinterpret_cast<uintptr_t>(p) & 15) == 0) {
            v = *reinterpret_cast<const v4i*>(p);
        } else {
            uint32_t h[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
#pragma unroll
            for (int c = 0; c < 8; ++c) if (k + c < K) h[c] = p[c];
            v = v4i{static_cast<int>(h[0] | (h[1] << 16)), static_cast<int>(h[2] | (h[3] << 16)),
                    static_cast<int>(h[4] | (h[5] << 16)), static_cast<int>(h[6] | (h[7] << 16))};
        }
    }
    return v;
}

// A stage is 64 k deep (four MFMA steps): with so little matrix work per element the loop is a chain of
// memory round trips, and a deeper stage makes it four times shorter.
constexpr int F16_BK = 64;
constexpr int F16_PITCH = F16_BK * 2 + 16;            // bytes per tile row: 16-byte fragment reads without bank conflicts

template <bool STREAM_C>
__global__ __launch_bounds__(256) void gemm_f16_kernel(const GemmParams p) {
    __shared__ __attribute__((aligned(16))) uint8_t lds_a[BM * F16_PITCH];
    __shared__ __attribute__((aligned(16))) uint8_t lds_b[BN * F16_PITCH];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int j = lane & 31, hh = lane >> 5;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
    int plane, m0, n0;
    tile_of_group(p, plane, m0, n0);                  // the launcher passes a single plane
    const uint16_t* A = reinterpret_cast<const uint16_t*>(p.A);
    const uint16_t* B = reinterpret_cast<const uint16_t*>(p.B);

    v16f acc[2][2];
#pragma unroll
    for (int ti = 0; ti < 2; ++ti)
#pragma unroll
        for (int tj = 0; tj < 2; ++tj)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[ti][tj][r] = 0.0f;

    // a thread's share of a 128 x 64 tile: row tid / 2, 32 consecutive k (four loads of 16 bytes)
    v4i ra[4], rb[4];
    const int srow = tid >> 1, sk = (tid & 1) * 32;
    const auto load_both = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            ra[i] = load_halves8(A, p.a_rs, m0 + srow, p.M, k0 + sk + 8 * i, p.K);
            rb[i] = load_halves8(B, p.b_rs, n0 + srow, p.N, k0 + sk + 8 * i, p.K);
        }
    };
    load_both(0);
    const int put = srow * F16_PITCH + sk * 2;
    const uint8_t* frag_a = lds_a + (wm + j) * F16_PITCH + hh * 16;
    const uint8_t* frag_b = lds_b + (wn + j) * F16_PITCH + hh * 16;

    for (int k0 = 0; k0 < p.K; k0 += F16_BK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            *reinterpret_cast<v4i*>(lds_a + put + 16 * i) = ra[i];
            *reinterpret_cast<v4i*>(lds_b + put + 16 * i) = rb[i];
        }
        __syncthreads();
        if (k0 + F16_BK < p.K) load_both(k0 + F16_BK);
#pragma unroll
        for (int s = 0; s < F16_BK / 16; ++s) {
            v8h fa[2], fb[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                fa[t] = *reinterpret_cast<const v8h*>(frag_a + t * 32 * F16_PITCH + s * 32);
                fb[t] = *reinterpret_cast<const v8h*>(frag_b + t * 32 * F16_PITCH + s * 32);
            }
#pragma unroll
            for (int ti = 0; ti < 2; ++ti)
#pragma unroll
                for (int tj = 0; tj < 2; ++tj)
                    acc[ti][tj] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[ti], fb[tj], acc[ti][tj], 0, 0, 0);
        }
        __syncthreads();
    }
    store_acc<false, STREAM_C, true, false>(p, p.C, acc, m0 + wm, n0 + wn, lane);
}

// The same contraction as a stream of tiles through resident work-groups whose waves divide the work: waves 4..7 only
// load (global -> registers, F16P_AHEAD stages of 64 k ahead, -> the other half of a double buffer in LDS) and waves
// 0..3 only read fragments, issue MFMAs and store finished tiles.  In gemm_f16_kernel every work-group of a round
// loads, contracts and stores at the same time as all the others, so the memory system sees a burst of loads and then
// a burst of stores, and a tile's four stages of K = 256 are four exposed round trips; here the loading waves run on
// into the next tile while the contracting waves store (they issue no loads, so nothing of theirs ever waits for a
// store), and a CU holds two such work-groups.  Tiles go to the XCDs in eight contiguous ranges, inside a range in
// bands of eight tile rows, so that the work-groups resident on an XCD at one time share operand panels in its L2.
// Same fragments, same order of the products, zero start and bias last as in gemm_f16_kernel: same bits.
// Conditions (the launcher's): K, both row pitches and both base addresses multiples of eight halves -- every load
// is sixteen bytes that lie inside one row or entirely past K --, operands and the dense output each below 2 GiB
// (buffer addressing: what lies outside reads as zero and is not stored), a grid that is a multiple of eight.
constexpr int F16P_AHEAD = 2;    // (three measured the same or 0.5 us slower: a longer start and end per work-group)
constexpr int F16P_STAGE = (BM + BN) * F16_PITCH;     // A's tile, then B's
template <bool STREAM_C>
__global__ __launch_bounds__(512, 2) void gemm_f16_pc_kernel(const GemmParams p, int total_tiles) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[2][F16P_STAGE];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool producer = wave >= 4;
    const int chunks = (p.K + F16_BK - 1) / F16_BK;

    // this work-group's tiles: first, first + step, ... below hi
    const int xcd = blockIdx.x & 7, step = gridDim.x >> 3;
    const int lo = static_cast<int>(static_cast<int64_t>(total_tiles) * xcd / 8);
    const int hi = static_cast<int>(static_cast<int64_t>(total_tiles) * (xcd + 1) / 8);
    const int first = lo + static_cast<int>(blockIdx.x >> 3);
    const int my_tiles = first < hi ? (hi - first + step - 1) / step : 0;
    const int total = my_tiles * chunks;              // stages this work-group contracts ...
    const int padded = (total + F16P_AHEAD - 1) / F16P_AHEAD * F16P_AHEAD;   // ... and passes
    const auto tile_origin = [&](int t, int& m0, int& n0) {
        const int band_rows = 8;
        const int band = t / (band_rows * p.tiles_n);
        t -= band * band_rows * p.tiles_n;
        const int rows_here = (p.tiles_m - band * band_rows) < band_rows ? (p.tiles_m - band * band_rows) : band_rows;
        m0 = (band * band_rows + t % rows_here) * BM;
        n0 = (t / rows_here) * BN;
    };

    // Both kinds of wave pass padded + 1 barriers: barrier g + 1 says "stage g is in LDS" and "stage g - 1 has been read".
    if (producer) {
        const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float*>(p.A), 0, static_cast<int>(((p.M - 1) * p.a_rs + p.K) * 2), 0x00020000);
        const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float*>(p.B), 0, static_cast<int>(((p.N - 1) * p.b_rs + p.K) * 2), 0x00020000);
        const uint32_t a_rs_bytes = static_cast<uint32_t>(p.a_rs) * 2u, b_rs_bytes = static_cast<uint32_t>(p.b_rs) * 2u;
        // a thread's share of a stage: rows ptid / 8 + 32 i of both tiles, eight halves from k = 8 (ptid % 8) on --
        // eight lanes read a row's 128 bytes
        const int ptid = tid & 255;
        const int prow = ptid >> 3, pk = (ptid & 7) * 8;
        const int put = prow * F16_PITCH + pk * 2;
        v4i ra[F16P_AHEAD][4], rb[F16P_AHEAD][4];
        int it = 0, ic = 0, m0 = 0, n0 = 0;             // the next stage to request: tile `it` of mine, stage ic of it
        if (my_tiles > 0) tile_origin(first, m0, n0);
        // (Past the last stage a request asks for nothing -- every offset outside -- but is still made: the count of
        // loads in flight that the wait for a stage names is then the same in every iteration, and the compiler
        // waits for that stage alone -- vmcnt(15) .. vmcnt(8) for its eight loads; with requests under a condition
        // it waited for all of them.)
        const auto request = [&](v4i (&xa)[4], v4i (&xb)[4]) {
            const int k = ic * F16_BK + pk;
            const uint32_t kb = static_cast<uint32_t>(k) * 2u;
            const bool live = it < my_tiles && k < p.K;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int ar = m0 + prow + 32 * i, br = n0 + prow + 32 * i;
                const uint32_t at = (live && ar < p.M) ? static_cast<uint32_t>(ar) * a_rs_bytes + kb : OUTSIDE;
                const uint32_t bt = (live && br < p.N) ? static_cast<uint32_t>(br) * b_rs_bytes + kb : OUTSIDE;
                xa[i] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, at, 0, 0));
                xb[i] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, bt, 0, 0));
            }
            if (++ic == chunks) {
                ic = 0;
                if (++it < my_tiles) tile_origin(first + it * step, m0, n0);
            }
        };
#pragma unroll
        for (int d = 0; d < F16P_AHEAD; ++d) { request(ra[d], rb[d]); __builtin_amdgcn_sched_barrier(0); }   // (in this order)
        // The register sets take turns by name: the loop body is written out F16P_AHEAD times, and runs whole -- the
        // stages past the last one move zeros, and the other waves pass their barriers (a way out of the middle of
        // the body joins the loop's back edge in the compiled code, and the wait at the loop's head then allows
        // for a set that has only just been requested: it waits for every load in flight).
        for (int g0 = 0; g0 < padded; g0 += F16P_AHEAD) {
#pragma unroll
            for (int d = 0; d < F16P_AHEAD; ++d) {
                const int g = g0 + d;
                uint8_t* half = lds[g & 1];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    *reinterpret_cast<v4i*>(half + put + i * 32 * F16_PITCH) = ra[d][i];
                    *reinterpret_cast<v4i*>(half + BM * F16_PITCH + put + i * 32 * F16_PITCH) = rb[d][i];
                }
                request(ra[d], rb[d]);
                __syncthreads();
            }
        }
        __syncthreads();                                // (the other waves' last stage)
    } else {
        const int j = lane & 31, hh = lane >> 5;
        const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
        const int frag_a = (wm + j) * F16_PITCH + hh * 16;
        const int frag_b = (BM + wn + j) * F16_PITCH + hh * 16;
        const __amdgpu_buffer_rsrc_t rsrc_c = __builtin_amdgcn_make_buffer_rsrc(p.C, 0, static_cast<int>(p.M * p.c_mi * 4), 0x00020000);
        __syncthreads();                                // stage 0 is in LDS
        int g = 0;
        for (int it = 0; it < my_tiles; ++it) {
            int m0, n0;
            tile_origin(first + it * step, m0, n0);
            float tail[2];
#pragma unroll
            for (int tj = 0; tj < 2; ++tj) {
                const int n = n0 + wn + tj * 32 + j;
                tail[tj] = (p.bias && n < p.N) ? p.bias[n] : 0.0f;
            }
            v16f acc[2][2];
#pragma unroll
            for (int ti = 0; ti < 2; ++ti)
#pragma unroll
                for (int tj = 0; tj < 2; ++tj)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[ti][tj][r] = 0.0f;
            for (int c = 0; c < chunks; ++c, ++g) {
                const uint8_t* half = lds[g & 1];
#pragma unroll
                for (int s = 0; s < F16_BK / 16; ++s) {
                    v8h fa[2], fb[2];
#pragma unroll
                    for (int t = 0; t < 2; ++t) {
                        fa[t] = *reinterpret_cast<const v8h*>(half + frag_a + t * 32 * F16_PITCH + s * 32);
                        fb[t] = *reinterpret_cast<const v8h*>(half + frag_b + t * 32 * F16_PITCH + s * 32);
                    }
#pragma unroll
                    for (int ti = 0; ti < 2; ++ti)
#pragma unroll
                        for (int tj = 0; tj < 2; ++tj)
                            acc[ti][tj] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[ti], fb[tj], acc[ti][tj], 0, 0, 0);
                }
                __syncthreads();                        // stage g has been read; stage g + 1 is in LDS
            }
            store_acc_buffer<STREAM_C, true>(rsrc_c, static_cast<uint32_t>(p.c_mi) * 4u, p.N, p.alpha, acc, m0 + wm, n0 + wn, lane, tail[0], tail[1]);
        }
        for (; g < padded; ++g) __syncthreads();
    }
}

// ------------------------------------------------------------------------------------------
// Large contractions split their operands once, ahead of the matrix work, instead of in every
// work-group that reads them (a 128-row panel of A is read by every tile column): the planes go to a
// workspace in the order the contraction consumes them,
//     [plane s][chunk of 16 k][tile of 32 rows][k half][row][8 bf16]   (1 KB per MFMA operand fragment)
// i.e. a fragment is stored lane by lane as the MFMA wants it (lane = 32 * (k half) + row, 16 bytes each).
// A work-group's share of one chunk is contiguous per plane, goes to LDS as it lies, and comes out of LDS
// with every lane reading its own 16 bytes of a 1 KB block: no bank conflicts either way, and a main loop
// of loads, LDS traffic and MFMAs only.
struct SplitJob {
    const float* src;
    uint8_t* dst;
    int rows, rows_pad, K, chunks;
    int64_t rs, ks;                                   // element (row, k) at src[row * rs + k * ks] ...
    int lm, lk;                                       // ... or, with lm > 0, at the compound address of LOAD_SPLIT_A
    int64_t mo, mi, ko, ki;
    int* fired;                                       // [rows_pad / 32]: set where a SplitGuard fired for that tile of 32 rows
};

template <bool KS1, bool COMPOUND>
__global__ __launch_bounds__(256) void split_operand_kernel(const SplitJob jb) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int kq = static_cast<int>(idx & 1);
    const int64_t rc = idx >> 1;
    const int row = static_cast<int>(rc % jb.rows_pad);
    const int c = static_cast<int>(rc / jb.rows_pad);
    if (c >= jb.chunks) return;
    const int kb = c * BK + kq * 8;
    v4f v[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    if (row < jb.rows) {
        if (COMPOUND) {
            const int64_t roff = static_cast<int64_t>(row / jb.lm) * jb.mo + static_cast<int64_t>(row % jb.lm) * jb.mi;
            const int kd = kb / jb.lk, kr = kb - kd * jb.lk;
            if (kr + 7 < jb.lk && kb + 7 < jb.K) {
                // the eight k share their outer index: one division for all of them
                const float* src = jb.src + roff + static_cast<int64_t>(kd) * jb.ko + static_cast<int64_t>(kr) * jb.ki;
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i >> 2][i & 3] = src[static_cast<int64_t>(i) * jb.ki];
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int k = kb + i;
                    if (k < jb.K) v[i >> 2][i & 3] = jb.src[roff + static_cast<int64_t>(k / jb.lk) * jb.ko + static_cast<int64_t>(k % jb.lk) * jb.ki];
                }
            }
        } else if (KS1) {
            const float* src = jb.src + static_cast<int64_t>(row) * jb.rs + kb;
            if (kb + 7 < jb.K) {
                v[0] = *reinterpret_cast<const v4f_u*>(src);
                v[1] = *reinterpret_cast<const v4f_u*>(src + 4);
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) if (kb + i < jb.K) v[i >> 2][i & 3] = src[i];
            }
        } else {
            const float* src = jb.src + static_cast<int64_t>(row) * jb.rs + static_cast<int64_t>(kb) * jb.ks;
#pragma unroll
            for (int i = 0; i < 8; ++i) if (kb + i < jb.K) v[i >> 2][i & 3] = src[static_cast<int64_t>(i) * jb.ks];
        }
    }
    uint2 lo[3], hi[3];
    SplitGuard guard;
    split4(v[0], lo, guard);
    split4(v[1], hi, guard);
#pragma unroll
    for (int s = 0; s < 3; ++s) {
        uint8_t* dst = jb.dst + ((static_cast<int64_t>(s) * jb.chunks + c) * jb.rows_pad + (row & ~31)) * 32 + kq * 512 + (row & 31) * 16;
        *reinterpret_cast<uint4*>(dst) = uint4{lo[s].x, lo[s].y, hi[s].x, hi[s].y};
    }
    if (guard.fired()) jb.fired[row >> 5] = 1;          // (rare; every writer writes the same value)
}

__global__ __launch_bounds__(256) void clear_flags_kernel(int* __restrict__ flags, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) flags[i] = 0;
}

// Work-group tile 256 x 128, four waves of 128 x 64 each (eight accumulator tiles): a fragment read from
// LDS feeds twice as many MFMAs as in the 64 x 64 arrangement, which had the LDS at three quarters of its bandwidth.
constexpr int PBM = 256;
constexpr int PLANES_MIN_TILES = 8;              // 128-wide tiles per side from which the operands are split ahead ...
constexpr int PLANES_MIN_GROUPS = 512;           // ... if that leaves two 256 x 128 work-groups for every CU
constexpr int PLANES_MIN_SLICE_CHUNKS = 16;      // a K slice is at least 256 long
template <bool SPLIT_C, bool STREAM_C>
__global__ __launch_bounds__(256, 2) void gemm_planes_kernel(const GemmParams p, const uint8_t* __restrict__ wa,
                                                             const uint8_t* __restrict__ wb, int chunks, int ma_pad, int nb_pad,
                                                             int slice_chunks, float* __restrict__ partial,
                                                             const int* __restrict__ fired_a, const int* __restrict__ fired_b) {
    constexpr int A_PLANE = PBM * 32, B_PLANE = BN * 32;      // fragments of 1 KB, no padding
    __shared__ __attribute__((aligned(16))) uint8_t lds_a[3 * A_PLANE];
    __shared__ __attribute__((aligned(16))) uint8_t lds_b[3 * B_PLANE];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int j = lane & 31;
    const int wm = (wave >> 1) * 128, wn = (wave & 1) * 64;

    // One plane only (the launcher's rule); the plane index of the tile numbering is the K slice: with
    // `partial` set, slice s contracts chunks [s * slice_chunks, (s + 1) * slice_chunks) and leaves its raw
    // sums in partial[s][m][n] for reduce_slices_kernel, so that skinny problems still fill the chip.
    int slice, m0, n0;
    tile_of_group<PBM>(p, slice, m0, n0);
    const int c_begin = slice * slice_chunks;
    const int c_end = c_begin + slice_chunks < chunks ? c_begin + slice_chunks : chunks;

    v16f acc[4][2];
#pragma unroll
    for (int tj = 0; tj < 2; ++tj) {
        const int n = n0 + wn + tj * 32 + j;
        const float b0 = (!partial && p.bias && n < p.N) ? p.bias[n] : 0.0f;
#pragma unroll
        for (int ti = 0; ti < 4; ++ti)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[ti][tj][r] = b0;
    }

    const size_t a_chunk = static_cast<size_t>(ma_pad) * 32, b_chunk = static_cast<size_t>(nb_pad) * 32;
    const size_t a_plane = a_chunk * chunks, b_plane = b_chunk * chunks;
    const uint8_t* ga = wa + static_cast<size_t>(m0) * 32 + tid * 16;
    const uint8_t* gb = wb + static_cast<size_t>(n0) * 32 + tid * 16;
    v4i ra[3][2], rb[3];
    const auto load_both = [&](int c) {
#pragma unroll
        for (int s = 0; s < 3; ++s) {
            ra[s][0] = *reinterpret_cast<const v4i*>(ga + s * a_plane + c * a_chunk);
            ra[s][1] = *reinterpret_cast<const v4i*>(ga + s * a_plane + c * a_chunk + 128 * 32);
            rb[s] = *reinterpret_cast<const v4i*>(gb + s * b_plane + c * b_chunk);
        }
    };
    load_both(c_begin);
    const int put = tid * 16;
    const uint8_t* frag_a = lds_a + wm * 32 + lane * 16;
    const uint8_t* frag_b = lds_b + wn * 32 + lane * 16;

    for (int c = c_begin; c < c_end; ++c) {
#pragma unroll
        for (int s = 0; s < 3; ++s) {
            *reinterpret_cast<v4i*>(lds_a + s * A_PLANE + put) = ra[s][0];
            *reinterpret_cast<v4i*>(lds_a + s * A_PLANE + 128 * 32 + put) = ra[s][1];
            *reinterpret_cast<v4i*>(lds_b + s * B_PLANE + put) = rb[s];
        }
        __syncthreads();
        if (c + 1 < c_end) load_both(c + 1);
        v8bf fb[2][3];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int s = 0; s < 3; ++s) fb[t][s] = *reinterpret_cast<const v8bf*>(frag_b + s * B_PLANE + t * 1024);
#pragma unroll
        for (int ti = 0; ti < 4; ++ti) {
            v8bf fa[3];
#pragma unroll
            for (int s = 0; s < 3; ++s) fa[s] = *reinterpret_cast<const v8bf*>(frag_a + s * A_PLANE + ti * 1024);
#pragma unroll
            for (int q = 0; q < 6; ++q)
#pragma unroll
                for (int tj = 0; tj < 2; ++tj)
                    acc[ti][tj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[SPLIT_TERMS[q][0]], fb[tj][SPLIT_TERMS[q][1]], acc[ti][tj], 0, 0, 0);
        }
        __syncthreads();
    }

    if (partial) {
        // raw sums, rows and columns padded to whole tiles: no bounds to check, 128 contiguous bytes per half-wave
        float* dst = partial + (static_cast<size_t>(slice) * ma_pad + m0 + wm) * nb_pad + n0 + wn + j;
#pragma unroll
        for (int ti = 0; ti < 4; ++ti)
#pragma unroll
            for (int tj = 0; tj < 2; ++tj)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    __builtin_nontemporal_store(acc[ti][tj][r], dst + static_cast<size_t>(ti * 32 + mfma32_row(r, lane)) * nb_pad + tj * 32);
        return;
    }
    // a tile of 32 rows of either operand that the split could not carry: this tile again, the reference's way
    // (the flags are the same for the whole work-group; with K slices reduce_slices_kernel looks at them instead)
    int fired = 0;
#pragma unroll
    for (int i = 0; i < PBM / 32; ++i) fired |= fired_a[(m0 >> 5) + i];
#pragma unroll
    for (int i = 0; i < BN / 32; ++i) fired |= fired_b[(n0 >> 5) + i];
    if (fired) {
        plain_tile(p, p.A, p.B, p.C, m0, n0, PBM, BN, tid);
        return;
    }
    store_acc<SPLIT_C, STREAM_C, false, false, 4>(p, p.C, acc, m0 + wm, n0 + wn, lane);
}

// C = alpha * (bias + sum over the K slices, in slice order) with the contraction's own output addressing
template <bool SPLIT_C>
__global__ __launch_bounds__(256) void reduce_slices_kernel(const GemmParams p, const float* __restrict__ partial,
                                                            int slices, int ma_pad, int nb_pad,
                                                            const int* __restrict__ fired_a, const int* __restrict__ fired_b) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int nq = (p.N + 3) / 4;
    const int m = static_cast<int>(idx / nq);
    const int n4 = static_cast<int>(idx - static_cast<int64_t>(m) * nq) * 4;
    if (m >= p.M) return;
    v4f sum = {0.f, 0.f, 0.f, 0.f};
    if (p.bias) {
#pragma unroll
        for (int c = 0; c < 4; ++c) if (n4 + c < p.N) sum[c] = p.bias[n4 + c];
    }
    const float* src = partial + static_cast<size_t>(m) * nb_pad + n4;          // nb_pad is a multiple of 128
    for (int s = 0; s < slices; ++s) sum += *reinterpret_cast<const v4f*>(src + static_cast<size_t>(s) * ma_pad * nb_pad);
    // operands the split could not carry: these four again, the reference's way -- by the flags of the splits, or
    // (callers that pass none) wherever the slices' sum is NaN, which is what a slice leaves for such a tile
    if (fired_a ? (fired_a[m >> 5] | fired_b[n4 >> 5]) != 0 : (sum[0] != sum[0] || sum[1] != sum[1] || sum[2] != sum[2] || sum[3] != sum[3])) {
#pragma unroll
        for (int c = 0; c < 4; ++c) if (n4 + c < p.N && (fired_a || sum[c] != sum[c])) sum[c] = plain_dot(p, p.A, p.B, m, n4 + c);
    }
    int64_t roff;
    if (SPLIT_C) roff = static_cast<int64_t>(m / p.c_lm) * p.c_mo + static_cast<int64_t>(m % p.c_lm) * p.c_mi;
    else         roff = static_cast<int64_t>(m) * p.c_mi;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const int n = n4 + c;
        if (n >= p.N) break;
        int64_t coff;
        if (SPLIT_C) coff = static_cast<int64_t>(n / p.c_ln) * p.c_no + static_cast<int64_t>(n % p.c_ln) * p.c_ni;
        else         coff = static_cast<int64_t>(n) * p.c_ni;
        p.C[roff + coff] = sum[c] * p.alpha;
    }
}

int launch_split(const SplitJob& jb, hipStream_t stream) {
    const int64_t threads = static_cast<int64_t>(jb.chunks) * jb.rows_pad * 2;
    const dim3 grid(static_cast<unsigned>((threads + 255) / 256)), block(256);
    if (jb.lm > 0)       hipLaunchKernelGGL((split_operand_kernel<false, true>), grid, block, 0, stream, jb);
    else if (jb.ks == 1) hipLaunchKernelGGL((split_operand_kernel<true, false>), grid, block, 0, stream, jb);
    else                 hipLaunchKernelGGL((split_operand_kernel<false, false>), grid, block, 0, stream, jb);
    return check_launch("split_operand_kernel");
}

// Which matrix pipe multiplies binary32 operands: 0 = the bf16 pipe through the exact three-way split (the
// default), 1 = the fp32 pipe (v_mfma_f32_32x32x2_f32, k ascending two at a time).  Set through
// ppml_hip_set_f32_arithmetic or, before the first contraction, by PPML_HIP_F32_ARITH=fp32 in the environment.
thread_local int t_f32_arithmetic = -1;            // per thread: callers with different wishes do not race

int f32_arithmetic() {
    if (t_f32_arithmetic < 0) {
        const char* env = std::getenv("PPML_HIP_F32_ARITH");
        t_f32_arithmetic = (env && std::strcmp(env, "fp32") == 0) ? 1 : 0;
    }
    return t_f32_arithmetic;
}

// `fixed_ws` / `fixed_cap`: a workspace the caller brings (the static array of the entry point that allocates
// nothing).  With one, the pool is never touched: a contraction that wants more workspace than `fixed_cap`
// is refused, one that wants none runs as it always does.
// How many K slices make `groups` output tiles come out even over the CUs (a CU's rate does not depend on how many
// work-groups it holds): the smallest count within 2 % of the best, slices of at least `least_chunks` chunks.
int even_slices(int groups, int chunks, int most_slices, int least_chunks = PLANES_MIN_SLICE_CHUNKS) {
    const int cus = device_cu_count();
    int most = chunks / least_chunks < most_slices ? chunks / least_chunks : most_slices;
    if (most < 1) most = 1;
    int slices = 1;
    double best = 1e30;
    for (int sl = 1; sl <= most; ++sl) {
        const int64_t wgs = static_cast<int64_t>(groups) * sl;
        const double waste = static_cast<double>((wgs + cus - 1) / cus * cus) / static_cast<double>(wgs);
        if (waste < best - 0.02) { best = waste; slices = sl; }
    }
    return slices;
}

// gemm_bf16x3_half_split_kernel for a single-plane contraction whose tall operand A has compound indices; -1 when the
// contraction is not of that kind (the caller goes on to the other forms).  p.tiles_m / p.tiles_n / p.stream_c are set.
int try_half_split(const GemmParams& p, hipStream_t stream, const char* what) {
    if (p.a_lm <= 0 || p.np2 * p.np3 != 1 || p.clamp || p.f16_in || !(p.c_lm >= p.M && p.c_ln >= p.N)) return -1;
    if (p.a_lk < BK || p.K % p.a_lk != 0 || p.tiles_n > 16 || p.tiles_m < 3) return -1;
    const bool gen = p.a_lk % BK != 0;                  // runs that are not whole chunks (that form: a span of at most 2^30 bytes)
    const int amode = p.a_ki == 1 ? HS_KRUN : p.a_mi == 1 ? HS_RRUN : -1;
    if (amode < 0) return -1;
    // 32-bit byte offsets: the tall operand's span and the dense output below 2 GiB
    const int64_t a_span = static_cast<int64_t>((p.M - 1) / p.a_lm) * p.a_mo + static_cast<int64_t>(p.a_lm - 1) * p.a_mi +
                           static_cast<int64_t>((p.K - 1) / p.a_lk) * p.a_ko + static_cast<int64_t>(p.a_lk - 1) * p.a_ki + 1;
    if (p.a_mo < 0 || p.a_mi < 0 || p.a_ko < 0 || p.a_ki < 0 || a_span * 4 >= (1LL << 31) || (gen && a_span * 4 > (1LL << 30))) return -1;
    const int chunks = (p.K + BK - 1) / BK;
    const int groups = p.tiles_m * p.tiles_n;
    int slices = even_slices(groups, chunks, 16);
    const int slice_chunks = (chunks + slices - 1) / slices;
    slices = (chunks + slice_chunks - 1) / slice_chunks;
    const int ma_pad = p.tiles_m * BM, nb_pad = p.tiles_n * BN;
    const size_t b_bytes = static_cast<size_t>(3) * chunks * nb_pad * 32;
    const size_t part_bytes = static_cast<size_t>(slices) * ma_pad * nb_pad * 4;
    const int n_flags = ma_pad / 32 + nb_pad / 32;
    const size_t flag_bytes = (static_cast<size_t>(n_flags) * 4 + 255) / 256 * 256;
    const Workspace held = workspace_take(b_bytes + part_bytes + flag_bytes, stream);
    uint8_t* ws = held.ptr;
    if (!ws) return -1;
    float* partial = reinterpret_cast<float*>(ws + b_bytes);
    int* fired_a = reinterpret_cast<int*>(ws + b_bytes + part_bytes);
    int* fired_b = fired_a + ma_pad / 32;
    GemmParams q = p;
    q.np2 = slices;                                      // the tile numbering walks the slices as planes
    const dim3 grid(static_cast<unsigned>(groups * slices)), block(512);
    hipLaunchKernelGGL(clear_flags_kernel, dim3((n_flags + 255) / 256), dim3(256), 0, stream, fired_a, n_flags);
    int rc = check_launch(what);
    const SplitJob jb{p.B, ws, p.N, nb_pad, p.K, chunks, p.b_rs, p.b_ks, 0, 0, 0, 0, 0, 0, fired_b};
    if (rc == RC_OK) rc = launch_split(jb, stream);
    if (rc == RC_OK) {
        const uint32_t span_bytes = static_cast<uint32_t>(a_span * 4);
#define PPML_HS(AMODE_, GEN_) hipLaunchKernelGGL((gemm_bf16x3_half_split_kernel<AMODE_, GEN_>), grid, block, 0, stream, q, ws, nb_pad, chunks, slice_chunks, \
                                                 partial, ma_pad, fired_a, span_bytes)
        if (amode == HS_KRUN) { if (gen) PPML_HS(HS_KRUN, true); else PPML_HS(HS_KRUN, false); }
        else                  { if (gen) PPML_HS(HS_RRUN, true); else PPML_HS(HS_RRUN, false); }
#undef PPML_HS
        rc = check_launch(what);
    }
    if (rc == RC_OK) {
        const int64_t threads = static_cast<int64_t>(p.M) * ((p.N + 3) / 4);
        hipLaunchKernelGGL((reduce_slices_kernel<false>), dim3(static_cast<unsigned>((threads + 255) / 256)), dim3(256), 0, stream, p, partial, slices,
                           ma_pad, nb_pad, fired_a, fired_b);
        rc = check_launch(what);
    }
    workspace_give(held, stream);
    return rc;
}

// gemm_bf16x3_pc_slices_kernel for a single dense plane with few output tiles under a long K; -1 when the contraction
// is not of that kind or no workspace is to be had (the caller goes on to the unsliced forms).
template <int MODE>
int try_pc_slices(const GemmParams& p, hipStream_t stream, const char* what) {
    const int chunks = (p.K + BK - 1) / BK;
    const int groups = p.tiles_m * p.tiles_n;
    // (two launches: about 10 us before the first chunk.  us over K for one to nine tiles, unsliced: 256 12, 400 16.5,
    // 512 20, 640 24, 752 27; in slices: 512 ... 1024 12.8-14, 2048 15-19)
    constexpr int LEAST = 6;                            // chunks a slice is long at least
    // (64 tiles of 128 x 128 under K = 512 measured 21.6 against 20.4 unsliced, under K = 640 22.7 against 24.3)
    if (p.np2 * p.np3 != 1 || groups * 2 > device_cu_count() || chunks < (groups * 4 <= device_cu_count() ? 4 * LEAST : 6 * LEAST)) return -1;
    int slices = even_slices(groups, chunks, 128, LEAST);
    if (slices < 2) return -1;
    const int slice_chunks = (chunks + slices - 1) / slices;
    slices = (chunks + slice_chunks - 1) / slice_chunks;
    const int ma_pad = p.tiles_m * BM, nb_pad = p.tiles_n * BN;
    const size_t part_bytes = static_cast<size_t>(slices) * ma_pad * nb_pad * 4;
    const Workspace held = workspace_take(part_bytes, stream);
    uint8_t* ws = held.ptr;
    if (!ws) return -1;
    float* partial = reinterpret_cast<float*>(ws);
    GemmParams q = p;
    q.np2 = slices;                                      // the tile numbering walks the slices as planes
    const dim3 grid(static_cast<unsigned>(groups * slices)), block(512);
    if (MODE == LOAD_K_CONTIG && p.K % 4 != 0)
        hipLaunchKernelGGL((gemm_bf16x3_pc_slices_kernel<MODE, false>), grid, block, 0, stream, q, chunks, slice_chunks, partial, ma_pad, nb_pad);
    else
        hipLaunchKernelGGL((gemm_bf16x3_pc_slices_kernel<MODE, true>), grid, block, 0, stream, q, chunks, slice_chunks, partial, ma_pad, nb_pad);
    int rc = check_launch(what);
    if (rc == RC_OK) {
        const int64_t threads = static_cast<int64_t>(p.M) * ((p.N + 3) / 4);
        hipLaunchKernelGGL((reduce_slices_kernel<false>), dim3(static_cast<unsigned>((threads + 255) / 256)), dim3(256), 0, stream, p, partial, slices,
                           ma_pad, nb_pad, static_cast<const int*>(nullptr), static_cast<const int*>(nullptr));
        rc = check_launch(what);
    }
    workspace_give(held, stream);
    return rc;
}

template <int MODE>
bool try_pc_slices_done(const GemmParams& p, hipStream_t stream, const char* what, int& rc) {
    rc = try_pc_slices<MODE>(p, stream, what);
    return rc >= 0;
}

int launch_gemm(GemmParams p, hipStream_t stream, const char* what, uint8_t* fixed_ws = nullptr, size_t fixed_cap = 0) {
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    // Streaming (non-temporal) stores where every store instruction writes whole 128-byte lines: dense rows of a
    // multiple of 32 floats, on a 128-byte boundary, in every plane.  Ordinary stores leave the output dirty in the
    // XCDs' L2s, which are written back when the kernel ends; streaming ones go out as they are issued.  Measured
    // on the attention-logit kernels (us, streaming / ordinary): 100 planes of 128 x 128  4.8 / 6.1, 400 of them
    // 8.0 / 10.9, 2000 of them 30.5 / 42.7, 824 planes of 256 x 256  49 / 54.  With rows that are not whole lines
    // it is the other way round at every size (412 planes of 103 x 103  12.3 / 10.0, 3200 of them 100 / 49:
    // partial lines are merged in L2 only by ordinary stores).  Outputs with compound addressing keep the older
    // rule (streaming from 128 MB on: 72 -> 63 us on the 216 MB logits at the time).
    {
        const bool compound = !(p.c_lm >= p.M && p.c_ln >= p.N);
        const bool planes_ok = (p.np2 == 1 || p.c_p2 % 32 == 0) && (p.np3 == 1 || p.c_p3 % 32 == 0);
        const bool whole_lines = !compound && p.c_ni == 1 && p.c_mi % 32 == 0 && p.N % 32 == 0 && planes_ok &&
                                 (reinterpret_cast<uintptr_t>(p.C) & 127) == 0;
        p.stream_c = compound ? static_cast<int64_t>(p.M) * p.N * p.np2 * p.np3 * 4 >= (128LL << 20) : whole_lines;
    }
    const int64_t total = static_cast<int64_t>(p.tiles_m) * p.tiles_n * p.np2 * p.np3;
    if (total <= 0 || total > 0x7fffffffLL) { set_error("%s: grid of %lld work-groups is out of range", what, (long long)total); return RC_BAD_ARGS; }
    const dim3 grid(static_cast<unsigned>(total)), block(256);
    const bool split = !(p.c_lm >= p.M && p.c_ln >= p.N);
    int mode = LOAD_STRIDED;
    if (p.a_ks == 1 && p.b_ks == 1) mode = LOAD_K_CONTIG;
    else if (p.a_rs == 1 && p.b_rs == 1) mode = LOAD_ROW_CONTIG;
    // Large single-plane contractions split their operands ahead of the matrix work (every element would
    // otherwise be split by each work-group that reads it).  Problems with few output tiles and a long K are
    // cut into K slices until two work-groups per CU have work; their partial sums are added in slice order
    // by a second kernel, so the result does not depend on scheduling.  When no workspace is to be had, the
    // call takes the same path as the small ones.
    const bool fp32_pipe = f32_arithmetic() == 1;
    const int64_t planes_groups = static_cast<int64_t>((p.M + PBM - 1) / PBM) * p.tiles_n;
    const int chunks = (p.K + BK - 1) / BK;
    int slices = 1;
    // (K slices are for problems that leave most CUs without a tile -- the outer-product-mean backward has 96 --; with
    // a tile per CU or so the split ahead of the matrix work costs more than the slices win: 26368 x 512 -> 256, 206
    // work-groups, took 107 us in two slices against 48 on operands split in the tile loop)
    if (planes_groups < PLANES_MIN_GROUPS / 4) {
        const int64_t want = (PLANES_MIN_GROUPS + planes_groups - 1) / planes_groups;
        const int64_t most = chunks / PLANES_MIN_SLICE_CHUNKS;
        slices = static_cast<int>(want < most ? want : most);
        if (slices < 1) slices = 1;
    }
    const bool planes_fit = slices > 1 ? planes_groups * slices >= PLANES_MIN_GROUPS / 2 && static_cast<int64_t>(p.M) * p.N >= (1 << 20)
                                       : p.tiles_m >= PLANES_MIN_TILES && p.tiles_n >= PLANES_MIN_TILES && planes_groups >= PLANES_MIN_GROUPS;
    if (!fp32_pipe && !fixed_ws && p.a_lm > 0) {
        const int rc = try_half_split(p, stream, what);
        if (rc >= 0) return rc;
    }
    if (!fp32_pipe && !p.clamp && !p.f16_in && p.np2 * p.np3 == 1 && planes_fit) {
        const int tiles_m = (p.M + PBM - 1) / PBM;
        const int ma_pad = tiles_m * PBM, nb_pad = p.tiles_n * BN;
        const int slice_chunks = (chunks + slices - 1) / slices;
        slices = (chunks + slice_chunks - 1) / slice_chunks;
        const size_t a_bytes = static_cast<size_t>(3) * chunks * ma_pad * 32, b_bytes = static_cast<size_t>(3) * chunks * nb_pad * 32;
        const size_t part_bytes = slices > 1 ? static_cast<size_t>(slices) * ma_pad * nb_pad * 4 : 0;
        const int n_flags = ma_pad / 32 + nb_pad / 32;  // one per tile of 32 rows of either operand (see SplitGuard)
        const size_t flag_bytes = (static_cast<size_t>(n_flags) * 4 + 255) / 256 * 256;
        const size_t ws_bytes = a_bytes + b_bytes + part_bytes + flag_bytes;
        uint8_t* ws = nullptr;
        Workspace held;
        if (fixed_ws) {
            if (ws_bytes > fixed_cap) {
                set_error("%s: this contraction needs %zu bytes of workspace, the static one holds %zu", what, ws_bytes, fixed_cap);
                return RC_BAD_ARGS;
            }
            ws = fixed_ws;
        } else {
            held = workspace_take(ws_bytes, stream);
            ws = held.ptr;
        }
        if (ws) {
            GemmParams q = p;
            q.tiles_m = tiles_m;
            q.np2 = slices;                              // the tile numbering walks the slices as planes
            float* partial = slices > 1 ? reinterpret_cast<float*>(ws + a_bytes + b_bytes) : nullptr;
            const dim3 pgrid(static_cast<unsigned>(q.tiles_m * q.tiles_n * slices));
            int* fired_a = reinterpret_cast<int*>(ws + a_bytes + b_bytes + part_bytes);
            int* fired_b = fired_a + ma_pad / 32;
            const SplitJob ja{p.A, ws, p.M, ma_pad, p.K, chunks, p.a_rs, p.a_ks, p.a_lm, p.a_lk, p.a_mo, p.a_mi, p.a_ko, p.a_ki, fired_a};
            const SplitJob jb{p.B, ws + a_bytes, p.N, nb_pad, p.K, chunks, p.b_rs, p.b_ks, 0, 0, 0, 0, 0, 0, fired_b};
            // (a small kernel, not a memset: this launcher may be recorded into a graph)
            hipLaunchKernelGGL(clear_flags_kernel, dim3((n_flags + 255) / 256), block, 0, stream, fired_a, n_flags);
            int rc = check_launch(what);
            if (rc == RC_OK) rc = launch_split(ja, stream);
            if (rc == RC_OK) rc = launch_split(jb, stream);
            if (rc == RC_OK) {
                const bool stream_c = p.stream_c && !partial;
                if (split && !partial) { if (stream_c) hipLaunchKernelGGL((gemm_planes_kernel<true, true>), pgrid, block, 0, stream, q, ws, ws + a_bytes, chunks, ma_pad, nb_pad, slice_chunks, partial, fired_a, fired_b);
                                         else hipLaunchKernelGGL((gemm_planes_kernel<true, false>), pgrid, block, 0, stream, q, ws, ws + a_bytes, chunks, ma_pad, nb_pad, slice_chunks, partial, fired_a, fired_b); }
                else                   { if (stream_c) hipLaunchKernelGGL((gemm_planes_kernel<false, true>), pgrid, block, 0, stream, q, ws, ws + a_bytes, chunks, ma_pad, nb_pad, slice_chunks, partial, fired_a, fired_b);
                                         else hipLaunchKernelGGL((gemm_planes_kernel<false, false>), pgrid, block, 0, stream, q, ws, ws + a_bytes, chunks, ma_pad, nb_pad, slice_chunks, partial, fired_a, fired_b); }
                rc = check_launch(what);
            }
            if (rc == RC_OK && partial) {
                const int64_t threads = static_cast<int64_t>(p.M) * ((p.N + 3) / 4);
                const dim3 rgrid(static_cast<unsigned>((threads + 255) / 256));
                if (split) hipLaunchKernelGGL((reduce_slices_kernel<true>), rgrid, block, 0, stream, p, partial, slices, ma_pad, nb_pad, fired_a, fired_b);
                else       hipLaunchKernelGGL((reduce_slices_kernel<false>), rgrid, block, 0, stream, p, partial, slices, ma_pad, nb_pad, fired_a, fired_b);
                rc = check_launch(what);
            }
            if (!fixed_ws) workspace_give(held, stream);
            return rc;
        }
    }
    // few tiles and a K loop worth it: the work-group divided into loading / splitting and contracting waves
    // (gemm_bf16x3_pc_kernel), where buffer addressing applies
    const bool two_sets = total <= device_cu_count() && p.K > 3 * BK;
#define PPML_LAUNCH_BF16(MODE, SPLIT)                                                                 \
    do {                                                                                              \
        if (p.stream_c) hipLaunchKernelGGL((gemm_bf16x3_kernel<MODE, SPLIT, true>), grid, block, 0, stream, p);  \
        else hipLaunchKernelGGL((gemm_bf16x3_kernel<MODE, SPLIT, false>), grid, block, 0, stream, p); \
    } while (0)
#define PPML_LAUNCH_F32(MODE, SPLIT)                                                                  \
    do {                                                                                              \
        if (p.stream_c) hipLaunchKernelGGL((gemm_f32_kernel<MODE, SPLIT, true>), grid, block, 0, stream, p);  \
        else hipLaunchKernelGGL((gemm_f32_kernel<MODE, SPLIT, false>), grid, block, 0, stream, p);    \
    } while (0)
    if (p.a_lm > 0) {
        if (split || p.f16_in || p.clamp) { set_error("%s: no split-operand instance for this addressing", what); return RC_BAD_ARGS; }
        if (fp32_pipe) PPML_LAUNCH_F32(LOAD_SPLIT_A, false);
        else PPML_LAUNCH_BF16(LOAD_SPLIT_A, false);
    }
    else if (!p.clamp && !p.f16_in && fp32_pipe) {
        if (mode == LOAD_K_CONTIG)        { if (split) PPML_LAUNCH_F32(LOAD_K_CONTIG, true);   else PPML_LAUNCH_F32(LOAD_K_CONTIG, false); }
        else if (mode == LOAD_ROW_CONTIG) { if (split) PPML_LAUNCH_F32(LOAD_ROW_CONTIG, true); else PPML_LAUNCH_F32(LOAD_ROW_CONTIG, false); }
        else                              { if (split) PPML_LAUNCH_F32(LOAD_STRIDED, true);    else PPML_LAUNCH_F32(LOAD_STRIDED, false); }
    }
    else if (!p.clamp && !p.f16_in && mode == LOAD_ROW_CONTIG && !split && p.c_ni == 1 && !p.bias &&
             p.K * p.a_ks * 4 < (1LL << 31) && p.K * p.b_ks * 4 < (1LL << 31) && p.M * p.c_mi * 4 < (1LL << 31) &&
             p.a_ks < (1 << 24) && p.b_ks < (1 << 24) && p.c_mi < (1 << 22)) {
        // (the last three keep "offset of a lane outside the matrix + up to 32 k steps / 128 rows" below 2^32)
        // contiguous rows, dense output planes below 2 GiB each: buffer addressing
        if (p.K <= 32) {
            // a short K: the persistent, single-stage form; two work-groups per CU, a multiple of eight in all
            // 128-wide tiles from about 100 rows a side (measured at the logit shapes: 103 rows 10.2 us against 10.6
            // with 64-wide tiles, 256 rows 43 against 47)
            const bool big = (p.M < p.N ? p.M : p.N) >= 96;
            const int tm = big ? 128 : 64;
            const int64_t tiles = static_cast<int64_t>((p.M + tm - 1) / tm) * ((p.N + tm - 1) / tm) * p.np2 * p.np3;
            if (tiles <= 0x7fffffffLL) {
                int wgs = (big ? 2 : 4) * device_cu_count();      // resident work-groups: 72 KB / 36 KB of LDS each
                if (tiles < wgs) wgs = static_cast<int>((tiles + 7) / 8 * 8);
                const dim3 pgrid(static_cast<unsigned>(wgs));
                // Rows that are not whole lines, dense, and one tile across: the tile leaves as one contiguous range.  It
                // costs an LDS round trip per tile, which pays once the output no longer stays in L2 anyway (us, ordinary
                // / contiguous: 100 planes of 103 x 103 4.9 / 6.1, 200 6.9 / 6.4, 412 10.0 / 8.0, 3200 50.7 / 43.9; 1200
                // planes of 50 x 50 9.5 / 9.7, 3000 18.6 / 17.8).
                const int64_t c_total = static_cast<int64_t>(p.M) * p.N * p.np2 * p.np3 * 4;
                const bool flat = !p.stream_c && p.c_mi == p.N && p.N <= tm && c_total >= (big ? 8LL << 20 : 24LL << 20);
                // Rows of whole lines that are longer than a tile is wide: through LDS too, sixteen bytes per lane (us,
                // registers as they lie / through LDS: 824 planes of 256 x 256 46-48 / 44.5, 200 of 512 x 512 45.4 / 41.5;
                // rows that one tile spans lose the round trip: 2000 planes of 128 x 128 30.2 / 31.4, 100 of them 4.8 / 5.5).
                const bool rows = p.stream_c && big && p.N > tm;
                const int form = rows ? C_ROWS : p.stream_c ? C_STREAM : flat ? C_FLAT : C_ORDINARY;
                // (the number of this launch: see lds_guard in the kernel)
                static std::atomic<uint64_t> launches{0};
                const uint64_t launch = launches.fetch_add(1, std::memory_order_relaxed) + 1;
                const uint32_t launch_mark = (static_cast<uint32_t>(launch) ^ static_cast<uint32_t>(launch >> 32)) * 0x9e3779b1u ^ 0x85ebca6bu;
#define PPML_SHORTK(TM_, FORM_) hipLaunchKernelGGL((gemm_bf16x3_shortk_kernel<TM_, FORM_>), pgrid, block, 0, stream, p, static_cast<int>(tiles), launch_mark)
                if (form == C_ROWS) PPML_SHORTK(128, C_ROWS);
                else if (big) { if (form == C_STREAM) PPML_SHORTK(128, C_STREAM); else if (form == C_FLAT) PPML_SHORTK(128, C_FLAT); else PPML_SHORTK(128, C_ORDINARY); }
                else     { if (form == C_STREAM) PPML_SHORTK(64, C_STREAM);  else if (form == C_FLAT) PPML_SHORTK(64, C_FLAT);  else PPML_SHORTK(64, C_ORDINARY); }
#undef PPML_SHORTK
                return check_launch(what);
            }
        }
        if (!fixed_ws) {
            const int rc = try_pc_slices<LOAD_ROW_CONTIG>(p, stream, what);
            if (rc >= 0) return rc;
        }
        if (p.K > 3 * BK && (p.N <= 32) != (p.M <= 32)) {
            // one narrow side: tiles of 128 x 32 along the other (gemm_bf16x3_pc_narrow_kernel)
            const bool side_n = p.N <= 32;
            const int64_t tiles_long = side_n ? p.tiles_m : p.tiles_n;
            if (side_n) p.tiles_n = 1; else p.tiles_m = 1;
            const dim3 ngrid(static_cast<unsigned>(tiles_long * p.np2 * p.np3));
#define PPML_RNARROW(SIDE_, STREAM_) hipLaunchKernelGGL((gemm_bf16x3_pc_narrow_kernel<LOAD_ROW_CONTIG, SIDE_, STREAM_, true>), ngrid, dim3(512), 0, stream, p)
            if (side_n) { if (p.stream_c) PPML_RNARROW(SIDE_N, true); else PPML_RNARROW(SIDE_N, false); }
            else        { if (p.stream_c) PPML_RNARROW(SIDE_M, true); else PPML_RNARROW(SIDE_M, false); }
#undef PPML_RNARROW
            return check_launch(what);
        }
        if (two_sets) {
            if (p.stream_c) hipLaunchKernelGGL((gemm_bf16x3_pc_kernel<LOAD_ROW_CONTIG, true, true>), grid, dim3(512), 0, stream, p);
            else hipLaunchKernelGGL((gemm_bf16x3_pc_kernel<LOAD_ROW_CONTIG, false, true>), grid, dim3(512), 0, stream, p);
        }
        else if (p.stream_c) hipLaunchKernelGGL((gemm_bf16x3_kernel<LOAD_ROW_CONTIG, false, true, true>), grid, block, 0, stream, p);
        else hipLaunchKernelGGL((gemm_bf16x3_kernel<LOAD_ROW_CONTIG, false, false, true>), grid, block, 0, stream, p);
    }
    else if (!p.clamp && !p.f16_in) {
        // binary32 operands without the finite guard: the contraction runs on the bf16 matrix pipe
        // rows contiguous in k, dense output planes, every plane below 2 GiB: buffer addressing (see load_kcontig_buffer)
        int slices_rc = -1;
        const bool k_fast = mode == LOAD_K_CONTIG && !split && p.c_ni == 1 && p.a_lm == 0 &&
                            ((p.M - 1) * p.a_rs + p.K) * 4 < (1LL << 31) && ((p.N - 1) * p.b_rs + p.K) * 4 < (1LL << 31) &&
                            p.M * p.c_mi * 4 < (1LL << 31) && p.c_mi < (1 << 22) && p.a_rs < (1 << 22) && p.b_rs < (1 << 22);
        // few tiles under a long K (a LinearLayer's weight gradient) go in K slices, whatever their width
        if (k_fast && !fixed_ws && try_pc_slices_done<LOAD_K_CONTIG>(p, stream, what, slices_rc)) return slices_rc;
        if (k_fast && p.K > 3 * BK && (p.N <= 32 || p.M <= 32)) {
            // one narrow side: tiles of 128 x 32 along the other (gemm_bf16x3_pc_narrow_kernel)
            const bool side_n = p.N <= 32;
            const int64_t tiles_long = side_n ? p.tiles_m : p.tiles_n;
            if (side_n) p.tiles_n = 1; else p.tiles_m = 1;
            const dim3 ngrid(static_cast<unsigned>(tiles_long * p.np2 * p.np3));
#define PPML_KNARROW(SIDE_, STREAM_, K4_) hipLaunchKernelGGL((gemm_bf16x3_pc_narrow_kernel<LOAD_K_CONTIG, SIDE_, STREAM_, K4_>), ngrid, dim3(512), 0, stream, p)
            const bool k4 = p.K % 4 == 0;
            if (side_n) { if (k4) { if (p.stream_c) PPML_KNARROW(SIDE_N, true, true); else PPML_KNARROW(SIDE_N, false, true); }
                          else    { if (p.stream_c) PPML_KNARROW(SIDE_N, true, false); else PPML_KNARROW(SIDE_N, false, false); } }
            else        { if (k4) { if (p.stream_c) PPML_KNARROW(SIDE_M, true, true); else PPML_KNARROW(SIDE_M, false, true); }
                          else    { if (p.stream_c) PPML_KNARROW(SIDE_M, true, false); else PPML_KNARROW(SIDE_M, false, false); } }
#undef PPML_KNARROW
        }
        else if (k_fast && two_sets) {
#define PPML_KPC(STREAM_, K4_) hipLaunchKernelGGL((gemm_bf16x3_pc_kernel<LOAD_K_CONTIG, STREAM_, K4_>), grid, dim3(512), 0, stream, p)
            if (p.K % 4 == 0) { if (p.stream_c) PPML_KPC(true, true); else PPML_KPC(false, true); }
            else              { if (p.stream_c) PPML_KPC(true, false); else PPML_KPC(false, false); }
#undef PPML_KPC
        }
        else if (k_fast) {
#define PPML_KFAST(STREAM_, K4_) hipLaunchKernelGGL((gemm_bf16x3_kernel<LOAD_K_CONTIG, false, STREAM_, true, K4_>), grid, block, 0, stream, p)
            if (p.K % 4 == 0) { if (p.stream_c) PPML_KFAST(true, true); else PPML_KFAST(false, true); }
            else              { if (p.stream_c) PPML_KFAST(true, false); else PPML_KFAST(false, false); }
#undef PPML_KFAST
        }
        // an output with compound addressing (the outer-product-mean in its graph and value forms) over operand planes
        // below 2 GiB that are contiguous in k or in their rows: buffer-addressed loads, the generic store
        else if (split && p.a_lm == 0 && mode == LOAD_K_CONTIG && ((p.M - 1) * p.a_rs + p.K) * 4 < (1LL << 31) &&
                 ((p.N - 1) * p.b_rs + p.K) * 4 < (1LL << 31) && p.a_rs < (1 << 22) && p.b_rs < (1 << 22)) {
#define PPML_KFAST_SPLIT(STREAM_, K4_) hipLaunchKernelGGL((gemm_bf16x3_kernel<LOAD_K_CONTIG, true, STREAM_, true, K4_>), grid, block, 0, stream, p)
            if (p.K % 4 == 0) { if (p.stream_c) PPML_KFAST_SPLIT(true, true); else PPML_KFAST_SPLIT(false, true); }
            else              { if (p.stream_c) PPML_KFAST_SPLIT(true, false); else PPML_KFAST_SPLIT(false, false); }
#undef PPML_KFAST_SPLIT
        }
        else if (split && p.a_lm == 0 && mode == LOAD_ROW_CONTIG && p.K * p.a_ks * 4 < (1LL << 31) && p.K * p.b_ks * 4 < (1LL << 31) &&
                 p.a_ks < (1 << 24) && p.b_ks < (1 << 24)) {
            if (p.stream_c) hipLaunchKernelGGL((gemm_bf16x3_kernel<LOAD_ROW_CONTIG, true, true, true>), grid, block, 0, stream, p);
            else hipLaunchKernelGGL((gemm_bf16x3_kernel<LOAD_ROW_CONTIG, true, false, true>), grid, block, 0, stream, p);
        }
        // A contiguous in k, B contiguous in its rows, dense output planes below 2 GiB (the backward of the triangle
        // multiplication): the loading / contracting form with a loader per operand, whatever the number of tiles
        else if (p.a_ks == 1 && p.b_rs == 1 && p.a_lm == 0 && !split && p.c_ni == 1 && p.K > BK &&
                 ((p.M - 1) * p.a_rs + p.K) * 4 < (1LL << 31) && p.K * p.b_ks * 4 < (1LL << 31) && p.M * p.c_mi * 4 < (1LL << 31) &&
                 p.c_mi < (1 << 22) && p.a_rs < (1 << 22) && p.b_ks < (1 << 24)) {
#define PPML_MIXED(STREAM_, K4_) hipLaunchKernelGGL((gemm_bf16x3_pc_kernel<LOAD_K_CONTIG, STREAM_, K4_, LOAD_ROW_CONTIG>), grid, dim3(512), 0, stream, p)
            if (p.K % 4 == 0) { if (p.stream_c) PPML_MIXED(true, true); else PPML_MIXED(false, true); }
            else              { if (p.stream_c) PPML_MIXED(true, false); else PPML_MIXED(false, false); }
#undef PPML_MIXED
        }
        else if (mode == LOAD_K_CONTIG)   { if (split) PPML_LAUNCH_BF16(LOAD_K_CONTIG, true);   else PPML_LAUNCH_BF16(LOAD_K_CONTIG, false); }
        else if (mode == LOAD_ROW_CONTIG) { if (split) PPML_LAUNCH_BF16(LOAD_ROW_CONTIG, true); else PPML_LAUNCH_BF16(LOAD_ROW_CONTIG, false); }
        else                              { if (split) PPML_LAUNCH_BF16(LOAD_STRIDED, true);    else PPML_LAUNCH_BF16(LOAD_STRIDED, false); }
    }
    else if (p.clamp) {
        if (split || p.f16_in) { set_error("%s: no clamped instance for this addressing", what); return RC_BAD_ARGS; }
        p.stream_c = 0;                                // (the clamped instances store the ordinary way, whatever the size)
        // planes of small contractions that leave most CUs without a 128 x 128 tile: 64 x 64 tiles, whole K at once
        const int64_t tiles64 = static_cast<int64_t>((p.M + 63) / 64) * ((p.N + 63) / 64) * p.np2 * p.np3;
        if (p.K <= MIDK_MAX && !p.bias && static_cast<int64_t>(grid.x) < 2 * device_cu_count() && tiles64 <= 0x7fffffffLL) {
            if (mode == LOAD_K_CONTIG) return launch_f32_midk<LOAD_K_CONTIG, true>(p, stream, what);
            if (mode == LOAD_ROW_CONTIG) return launch_f32_midk<LOAD_ROW_CONTIG, true>(p, stream, what);
        }
        if (mode == LOAD_K_CONTIG) hipLaunchKernelGGL((gemm_f32_kernel<LOAD_K_CONTIG, false, false, true>), grid, block, 0, stream, p);
        else if (mode == LOAD_ROW_CONTIG) hipLaunchKernelGGL((gemm_f32_kernel<LOAD_ROW_CONTIG, false, false, true>), grid, block, 0, stream, p);
        else hipLaunchKernelGGL((gemm_f32_kernel<LOAD_STRIDED, false, false, true>), grid, block, 0, stream, p);
    }
    else {
        if (split || p.np2 * p.np3 != 1 || p.a_ks != 1 || p.b_ks != 1) { set_error("%s: no F16 instance for this addressing", what); return RC_BAD_ARGS; }
        // the streaming form where every load is sixteen aligned bytes and 32-bit offsets reach everything
        const bool aligned8 = p.K % 8 == 0 && p.a_rs % 8 == 0 && p.b_rs % 8 == 0 &&
                              ((reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.B)) & 15) == 0;
        const bool in_reach = ((p.M - 1) * p.a_rs + p.K) * 2 < (1LL << 31) && ((p.N - 1) * p.b_rs + p.K) * 2 < (1LL << 31) &&
                              p.c_ni == 1 && p.M * p.c_mi * 4 < (1LL << 31) && p.c_mi < (1 << 22);
        if (aligned8 && in_reach) {
            const int64_t resident = 2LL * device_cu_count() / 8 * 8;      // two work-groups per CU (LDS: 72 KB each)
            const int64_t wgs = std::max<int64_t>(8, std::min<int64_t>((total + 7) / 8 * 8, resident));
            const dim3 pgrid(static_cast<unsigned>(wgs));
            if (p.stream_c) hipLaunchKernelGGL((gemm_f16_pc_kernel<true>), pgrid, dim3(512), 0, stream, p, static_cast<int>(total));
            else hipLaunchKernelGGL((gemm_f16_pc_kernel<false>), pgrid, dim3(512), 0, stream, p, static_cast<int>(total));
        }
        else if (p.stream_c) hipLaunchKernelGGL((gemm_f16_kernel<true>), grid, block, 0, stream, p);
        else hipLaunchKernelGGL((gemm_f16_kernel<false>), grid, block, 0, stream, p);
    }
#undef PPML_LAUNCH_BF16
#undef PPML_LAUNCH_F32
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

extern "C" int ppml_hip_set_f32_arithmetic(int mode) {
    const int before = f32_arithmetic();
    if (mode == 0 || mode == 1) t_f32_arithmetic = mode;
    return before;
}

extern "C" int mul_mat_hip(const float* A, const float* B, float* C, int M, int K, int N,
                           const float* bias, ppml_hip_stream_t stream) {
    if (!A || !B || !C || M <= 0 || K <= 0 || N <= 0) { set_error("mul_mat_hip: bad arguments (M=%d K=%d N=%d)", M, K, N); return RC_BAD_ARGS; }
    StatsScope stat("hip/mul_mat", M, K, N, static_cast<hipStream_t>(stream));
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
    StatsScope stat("hip/mul_mat-f16", M, K, N, static_cast<hipStream_t>(stream));
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
    StatsScope stat("hip/mul_mat-tn", M, K, Nc, static_cast<hipStream_t>(stream));
    GemmParams p = plain_params();
    p.A = A; p.B = Bm; p.C = O;
    p.M = M; p.N = Nc; p.K = K;
    p.a_rs = 1; p.a_ks = M; p.b_rs = 1; p.b_ks = Nc;
    p.c_mi = Nc; p.c_ni = 1;
    p.alpha = alpha;
    return launch_gemm(p, static_cast<hipStream_t>(stream), "mul_mat_tn_hip");
}

// ---- the entry point that allocates nothing -------------------------------------------------------------
// Workspace of mul_mat_tn_noalloc_hip: the split planes (and K-slice partial sums) that mul_mat_tn_hip takes
// from the stream-ordered pool live here instead, for callers that may not allocate (HIP graph capture, tight
// serving loops).  Every device the library runs on holds its own copy until the process ends.  The name below
// is a host-side stand-in for the symbol, not a device address: host code uses the per-device pointer that
// hipGetSymbolAddress returned, never the name.
constexpr size_t NOALLOC_SCRATCH_BYTES = static_cast<size_t>(64) << 20;
static __device__ __align__(256) uint8_t scratch[NOALLOC_SCRATCH_BYTES];

namespace ppmlhip {
namespace {
constexpr int NOALLOC_MAX_DEVICES = 64;
std::mutex g_scratch_mu;
uint8_t* g_scratch_ptr[NOALLOC_MAX_DEVICES];          // per device: each GPU has the array at its own address
}  // namespace

// Looks the array's address up on the current device (once per device); called by ppml_hip_init with the
// device it has just selected, and by the entry point for a device nobody initialised.
int noalloc_scratch_setup(uint8_t** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= NOALLOC_MAX_DEVICES) {
        (void)hipGetLastError();
        set_error("mul_mat_tn_noalloc_hip: no current device below %d", NOALLOC_MAX_DEVICES);
        return RC_NO_DEVICE;
    }
    std::lock_guard<std::mutex> guard(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            (void)hipGetLastError();
            set_error("mul_mat_tn_noalloc_hip: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
            return RC_NO_DEVICE;
        }
        g_scratch_ptr[dev] = static_cast<uint8_t*>(ptr);
    }
    if (out) *out = g_scratch_ptr[dev];
    return RC_OK;
}
}  // namespace ppmlhip

extern "C" int mul_mat_tn_noalloc_hip(const float* A, const float* Bm, float* O, int M, int K, int Nc, float alpha,
                                      ppml_hip_stream_t stream) {
    if (!A || !Bm || !O || M <= 0 || K <= 0 || Nc <= 0) { set_error("mul_mat_tn_noalloc_hip: bad arguments"); return RC_BAD_ARGS; }
    uint8_t* ws = nullptr;
    const int rc = noalloc_scratch_setup(&ws);
    if (rc != RC_OK) return rc;
    GemmParams p = plain_params();
    p.A = A; p.B = Bm; p.C = O;
    p.M = M; p.N = Nc; p.K = K;
    p.a_rs = 1; p.a_ks = M; p.b_rs = 1; p.b_ks = Nc;
    p.c_mi = Nc; p.c_ni = 1;
    p.alpha = alpha;
    // No statistics scope here: its events would be created on the way.  Nothing in the workspace has to start
    // at zero: the split kernels write every byte of the planes they hand on (padding rows and k included) and
    // every K slice writes its whole padded block of partial sums before they are added.
    return launch_gemm(p, static_cast<hipStream_t>(stream), "mul_mat_tn_noalloc_hip", ws, NOALLOC_SCRATCH_BYTES);
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
    StatsScope stat("hip/out_prod", ne1, ne01, ne0, static_cast<hipStream_t>(stream));
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

// out_prod of the two {1,0,2,3} permutations of src0 and src1, without the permutations: the contraction runs
// over the INNERMOST dimension of both operands as they lie,
//     dst[i0, i1, i2, i3] = sum_k src0[k, i0, i2 / (ne2 / ne02), i3 / (ne3 / ne03)] * src1[k, i1, i2, i3],
// which is what the second contraction of the attention chain asks for (src/modules/Attention.cpp:277-281:
// out_prod(permute(attn), permute(V)), attn [Lk, Lq, h, B], V [L, D, h, B]).  The same kernel as out_prod_hip with
// the operands read k-contiguous instead of row-contiguous: same products, same order, same bits.
extern "C" int out_prod_tt_hip(const float* src0, const float* src1, float* dst,
                               int64_t ne00, int64_t ne01, int64_t ne02, int64_t ne03,
                               int64_t ne10, int64_t ne11, int64_t ne12, int64_t ne13,
                               int64_t ne0, int64_t ne1, int64_t ne2, int64_t ne3,
                               ppml_hip_stream_t stream) {
    if (!src0 || !src1 || !dst) { set_error("out_prod_tt_hip: null pointer"); return RC_BAD_ARGS; }
    const bool pos = ne00 > 0 && ne01 > 0 && ne02 > 0 && ne03 > 0 && ne10 > 0 && ne11 > 0 && ne12 > 0 && ne13 > 0;
    if (!pos || ne00 != ne10 || ne0 != ne01 || ne1 != ne11 || ne2 != ne12 || ne3 != ne13 ||
        ne2 % ne02 != 0 || ne3 % ne03 != 0 || ne0 > 0x7fffffff || ne1 > 0x7fffffff || ne00 > 0x7fffffff) {
        set_error("out_prod_tt_hip: shape mismatch src0[%lld,%lld,%lld,%lld] src1[%lld,%lld,%lld,%lld] dst[%lld,%lld,%lld,%lld]",
                  (long long)ne00, (long long)ne01, (long long)ne02, (long long)ne03,
                  (long long)ne10, (long long)ne11, (long long)ne12, (long long)ne13,
                  (long long)ne0, (long long)ne1, (long long)ne2, (long long)ne3);
        return RC_BAD_ARGS;
    }
    StatsScope stat("hip/out_prod", ne1, ne00, ne0, static_cast<hipStream_t>(stream));
    GemmParams p = plain_params();
    p.A = src1; p.B = src0; p.C = dst;                 // rows = i1 (src1), cols = i0 (src0)
    p.M = static_cast<int>(ne1); p.N = static_cast<int>(ne0); p.K = static_cast<int>(ne00);
    p.a_rs = ne10; p.a_ks = 1; p.b_rs = ne00; p.b_ks = 1;
    p.np2 = static_cast<int>(ne2); p.np3 = static_cast<int>(ne3);
    p.a_p2 = ne10 * ne11; p.a_p3 = ne10 * ne11 * ne12;
    p.b_p2 = ne00 * ne01; p.b_p3 = ne00 * ne01 * ne02;
    p.c_p2 = ne0 * ne1;   p.c_p3 = ne0 * ne1 * ne2;
    p.b_div2 = static_cast<int>(ne2 / ne02); p.b_div3 = static_cast<int>(ne3 / ne03);
    p.c_mi = ne0; p.c_ni = 1;
    return launch_gemm(p, static_cast<hipStream_t>(stream), "out_prod_tt_hip");
}

extern "C" int outer_prod_mean_hip(const float* left, const float* right, float* dst,
                                   int64_t D, int64_t L, int64_t N, int64_t B, float inv_N,
                                   ppml_hip_stream_t stream) {
    if (!left || !right || !dst || D <= 0 || L <= 0 || N <= 0 || B <= 0 || D * L > 0x7fffffff || N > 0x7fffffff) {
        set_error("outer_prod_mean_hip: bad arguments"); return RC_BAD_ARGS;
    }
    StatsScope stat("hip/outer_prod_mean", D * L, N, D * L, static_cast<hipStream_t>(stream));
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
    StatsScope stat("hip/outer_product_mean-value", D * L, N, D * L, static_cast<hipStream_t>(stream));
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
    StatsScope stat("hip/tri_mul", I, K, J, static_cast<hipStream_t>(stream));
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
        StatsScope stat("hip/tri_mul_back", M, Kc, N, static_cast<hipStream_t>(stream));
        GemmParams p = plain_params();
        // an output whose ROW index runs along memory is the dense plane of the transposed product: the operands trade
        // places (the fast forms of the contraction store dense planes)
        const bool swap = c_mi == 1 && c_ni != 1;
        p.A = swap ? b : a; p.B = swap ? a : b; p.C = c;
        p.M = static_cast<int>(swap ? N : M); p.N = static_cast<int>(swap ? M : N); p.K = static_cast<int>(Kc);
        p.a_rs = (swap ? b_rs : a_rs) * B; p.a_ks = (swap ? b_ks : a_ks) * B;
        p.b_rs = (swap ? a_rs : b_rs) * B; p.b_ks = (swap ? a_ks : b_ks) * B;
        p.c_mi = (swap ? c_ni : c_mi) * B; p.c_ni = (swap ? c_mi : c_ni) * B;
        p.np2 = static_cast<int>(B); p.np3 = static_cast<int>(D);
        p.a_p2 = 1; p.b_p2 = 1; p.c_p2 = 1;
        p.a_p3 = (swap ? b_p3 : a_p3) * B; p.b_p3 = (swap ? a_p3 : b_p3) * B; p.c_p3 = c_p3 * B;
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
        StatsScope stat("hip/outer_prod_mean_back", D * L, D * L, N, static_cast<hipStream_t>(stream));
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
