// Q8_0 path for gfx950: row quantizer, dequantizer, weight repack and the fused
// quantize + int8-MFMA linear kernel.
//
// Reference behaviour restated here (paths relative to the reference tree):
//   quantizer arithmetic     include/ppml/QuantBlocks.h:62-79
//   block dot and settlement src/cuda/MulMatQ8Kernel.cu:120-142
//   launcher contract        src/cuda/MulMatQ8Kernel.cu:476-547, src/cuda/QuantKernels.cu:86-109
#include "common.hpp"

namespace ppmlhip {
namespace {

// ------------------------------------------------------------------------------------------
// Quantizer arithmetic shared by the standalone and the fused kernel.
// ------------------------------------------------------------------------------------------

// max over each aligned group of 8 lanes (one Q8 block when every lane holds 4 elements)
__device__ __forceinline__ float group8_max(float v) {
    float o;
    o = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, false));  // lane ^ 1
    v = fmaxf(v, o);
    o = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, false));  // lane ^ 2
    v = fmaxf(v, o);
    o = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, false)); // 7 - lane (half row mirror)
    v = fmaxf(v, o);
    return v;
}

struct BlockQuant {
    uint32_t q4;      // this lane's 4 quants, element c in byte c
    uint16_t d_bits;  // fp16 scale of the block
};

// x holds elements 4*c8 .. 4*c8+3 of one 32-element block, the 8 lanes of an aligned group hold
// the whole block.  IEEE division, round half away from zero, clamp to +-127.
__device__ __forceinline__ BlockQuant quantize_block_lane(v4f x) {
    float amax = 0.0f;
    amax = fmaxf(amax, fabsf(x[0]));   // fmaxf drops NaN like std::fmax
    amax = fmaxf(amax, fabsf(x[1]));
    amax = fmaxf(amax, fabsf(x[2]));
    amax = fmaxf(amax, fabsf(x[3]));
    amax = group8_max(amax);
    const float d = amax / 127.0f;
    const float inv = (amax == 0.0f) ? 0.0f : 1.0f / d;
    BlockQuant out;
    out.d_bits = __half_as_ushort(__float2half_rn(d));
    uint32_t packed = 0;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        float q = roundf(x[c] * inv);
        q = q > 127.0f ? 127.0f : (q < -127.0f ? -127.0f : q);
        packed |= (static_cast<uint32_t>(static_cast<int>(q)) & 0xffu) << (8 * c);
    }
    out.q4 = packed;
    return out;
}

__device__ __forceinline__ float half_bits_to_float(uint16_t h) {
    return __half2float(__ushort_as_half(h));
}

// ------------------------------------------------------------------------------------------
// Standalone row quantizer / dequantizer (interleaved 34-byte blocks in HBM)
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void quantize_rows_q8_0_kernel(const float* __restrict__ x,
                                                                 uint8_t* __restrict__ y,
                                                                 int64_t nblocks) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    int64_t ib = t >> 3;
    const int c8 = static_cast<int>(t & 7);
    const bool live = ib < nblocks;
    if (!live) ib = nblocks - 1;                       // keep the whole 8-lane group convergent
    const v4f xv = *reinterpret_cast<const v4f_u*>(x + ib * QK + c8 * 4);
    const BlockQuant bq = quantize_block_lane(xv);
    if (!live) return;
    uint8_t* blk = y + ib * Q8_0_BYTES;               // 2-byte aligned only
    uint16_t* q16 = reinterpret_cast<uint16_t*>(blk + 2 + c8 * 4);
    q16[0] = static_cast<uint16_t>(bq.q4 & 0xffffu);
    q16[1] = static_cast<uint16_t>(bq.q4 >> 16);
    if (c8 == 0) *reinterpret_cast<uint16_t*>(blk) = bq.d_bits;
}

__global__ __launch_bounds__(256) void dequantize_q8_0_kernel(const uint8_t* __restrict__ x,
                                                              float* __restrict__ y, int64_t ne) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= ne) return;
    const int64_t ib = i / QK;
    const int iq = static_cast<int>(i - ib * QK);
    const uint8_t* blk = x + ib * Q8_0_BYTES;
    const float d = half_bits_to_float(*reinterpret_cast<const uint16_t*>(blk));
    y[i] = d * static_cast<float>(static_cast<int8_t>(blk[2 + iq]));
}

// ------------------------------------------------------------------------------------------
// Weight fragments.
//
// One int8 MFMA 32x32x32 consumes, per lane, 16 consecutive quants of one weight row:
// lane l -> row 32*ct + (l & 31), quants 16*(l >> 5) .. +15 of block b.  The activation operand
// is laid out the same way, so whatever order the instruction walks K in, equal K meets equal K.
//
// PPML_WTYPE_Q8_0M stores exactly these fragments: for tile ct and block b the 64 lanes' 16
// bytes are consecutive (1 KiB), followed by one fp16 scale plane [ct][b][32].  The tile count is
// rounded up to even and rows beyond M are zero, so kernels need no guard on the weight side.
// ------------------------------------------------------------------------------------------
__host__ __device__ inline int packed_tiles(int M) { return (((M + 31) / 32) + 1) & ~1; }

struct WGeom {
    const uint8_t* W;
    int M, nblk, mct_pad;
};

// 16 quants of weight row 32*ct + (lane & 31), k-half lane >> 5, block b
template <int WT>
__device__ __forceinline__ v4i load_wq(const WGeom& g, int ct, int b, int lane) {
    if (WT == PPML_WTYPE_Q8_0M) {
        ct = ct < g.mct_pad ? ct : g.mct_pad - 1;     // tiles past the end repeat the last one; never stored
        const int64_t frag = static_cast<int64_t>(ct) * g.nblk + b;
        return *reinterpret_cast<const v4i*>(g.W + (frag * 64 + lane) * 16);
    }
    const int hh = lane >> 5;
    int m = ct * 32 + (lane & 31);
    m = m < g.M ? m : g.M - 1;                        // rows past the end repeat the last one; never stored
    const int64_t blk = static_cast<int64_t>(m) * g.nblk + b;
    v4i q;
    if (WT == PPML_WTYPE_Q8_0R) {
        typedef int v4i_u __attribute__((ext_vector_type(4), aligned(4)));
        q = *reinterpret_cast<const v4i_u*>(g.W + blk * 32 + hh * 16);
    } else if (WT == PPML_WTYPE_Q8_0) {
        const uint16_t* q16 = reinterpret_cast<const uint16_t*>(g.W + blk * Q8_0_BYTES + 2 + hh * 16);  // 2-byte aligned
#pragma unroll
        for (int c = 0; c < 4; ++c)
            q[c] = static_cast<int>(static_cast<uint32_t>(q16[2 * c]) | (static_cast<uint32_t>(q16[2 * c + 1]) << 16));
    } else {                                           // Q8_1: {half d; half s; int8 qs[32]}, 4-byte aligned
        const int* q32 = reinterpret_cast<const int*>(g.W + blk * Q8_1_BYTES + 4 + hh * 16);
#pragma unroll
        for (int c = 0; c < 4; ++c) q[c] = q32[c];
    }
    return q;
}

// fp16 scale bits of weight row 32*ct + (lane & 31), block b
template <int WT>
__device__ __forceinline__ uint16_t load_wd(const WGeom& g, int ct, int b, int lane) {
    if (WT == PPML_WTYPE_Q8_0M) {
        ct = ct < g.mct_pad ? ct : g.mct_pad - 1;
        const uint16_t* dplane = reinterpret_cast<const uint16_t*>(g.W + static_cast<int64_t>(g.mct_pad) * g.nblk * 1024);
        return dplane[(static_cast<int64_t>(ct) * g.nblk + b) * 32 + (lane & 31)];
    }
    int m = ct * 32 + (lane & 31);
    m = m < g.M ? m : g.M - 1;
    const int64_t blk = static_cast<int64_t>(m) * g.nblk + b;
    if (WT == PPML_WTYPE_Q8_0R) {
        const uint16_t* dplane = reinterpret_cast<const uint16_t*>(g.W + static_cast<int64_t>(g.M) * g.nblk * 32);
        return dplane[blk];
    }
    const int stride = (WT == PPML_WTYPE_Q8_0) ? Q8_0_BYTES : Q8_1_BYTES;
    return *reinterpret_cast<const uint16_t*>(g.W + blk * stride);
}

template <int WT>
__global__ __launch_bounds__(64) void q8_weight_pack_kernel(const uint8_t* __restrict__ W,
                                                            uint8_t* __restrict__ out, int M, int nblk,
                                                            int mct_pad) {
    const int frag = blockIdx.x;                       // ct * nblk + b
    const int ct = frag / nblk, b = frag - ct * nblk;
    const int lane = threadIdx.x;
    const WGeom g{W, M, nblk, mct_pad};
    const bool live = ct * 32 + (lane & 31) < M;
    v4i q = load_wq<WT>(g, ct, b, lane);
    uint16_t d = load_wd<WT>(g, ct, b, lane);
    if (!live) { q = v4i{0, 0, 0, 0}; d = 0; }
    *reinterpret_cast<v4i*>(out + (static_cast<int64_t>(frag) * 64 + lane) * 16) = q;
    if (lane < 32) {
        uint16_t* dplane = reinterpret_cast<uint16_t*>(out + static_cast<int64_t>(mct_pad) * nblk * 1024);
        dplane[static_cast<int64_t>(frag) * 32 + lane] = d;
    }
}

// ------------------------------------------------------------------------------------------
// Fused Q8_0 linear:  C = Q8_0(X) . W^T   for one tile of 32 activation rows per work-group.
//
//   phase 1  the work-group streams its 32 x K slice of X once from HBM (16-byte loads, 8 lanes
//            per Q8 block, block absmax by DPP), quantizes it and leaves it in LDS already in
//            MFMA-fragment order, scales beside it as f32.  Nothing quantized goes back to HBM.
//   phase 2  wave w owns P consecutive 32-column tiles of the output (P even).  For every block
//            b (ascending) and every pair of tiles it issues two v_mfma_i32_32x32x32_i8 -> exact
//            int32 block sums, and one v_mfma_f32_32x32x1_2b_f32 whose two 32x32 outer products
//            are the scale products d_a[row]*d_w[col] of both tiles (each the exact product of two
//            halves), then settles acc = fma(float(sumi), d_w*d_a, acc) on the VALU.  The weight
//            fragments of block b+1 are requested as soon as the MFMAs of block b have read theirs.
//   phase 3  each half-wave store instruction writes one full 128-byte line of a C row.
//
// LDS per work-group: KC * 1152 bytes (KC = blocks staged at once, at most 32).
// ------------------------------------------------------------------------------------------
constexpr int TILE_TOK = 32;
constexpr int KC_MAX = 32;          // blocks of K staged in LDS at once (K = 1024 per chunk)
constexpr int UB = 4;               // quantizer units (8 rows x 1 block) a wave keeps in flight

typedef float v32f __attribute__((ext_vector_type(32)));

// Read cursor over the weight data of one pair of column tiles (ct, ct+1): 32-bit byte offsets
// from the weight base, advanced by a fixed stride per Q8 block.
template <int WT>
struct WPair {
    uint32_t oq0, oq1, od;   // offsets of this lane's fragment of tile ct, of tile ct+1, and of its scale
    v4i q0, q1;              // fragments of block b
    uint32_t d_bits;         // fp16 scale of tile ct (lanes 0-31) / ct+1 (lanes 32-63); converted at use

    static constexpr uint32_t q_stride() {
        return WT == PPML_WTYPE_Q8_0M ? 1024u : WT == PPML_WTYPE_Q8_0R ? 32u : WT == PPML_WTYPE_Q8_0 ? 34u : 36u;
    }
    static constexpr uint32_t d_stride() {
        return WT == PPML_WTYPE_Q8_0M ? 64u : WT == PPML_WTYPE_Q8_0R ? 2u : WT == PPML_WTYPE_Q8_0 ? 34u : 36u;
    }
    __device__ __forceinline__ void init(const WGeom& g, int ct, int lane) {
        const uint32_t j = lane & 31, hh = lane >> 5;
        const uint32_t nblk = g.nblk;
        if (WT == PPML_WTYPE_Q8_0M) {
            // tiles past the end repeat the last pair; their results are never stored
            const uint32_t c = ct + 1 < g.mct_pad ? ct : g.mct_pad - 2;
            oq0 = (c * nblk * 64u + lane) * 16u;
            oq1 = oq0 + nblk * 1024u;
            od = static_cast<uint32_t>(g.mct_pad) * nblk * 1024u + ((c + hh) * nblk * 32u + j) * 2u;
            return;
        }
        // rows past the end repeat the last row; their results are never stored
        uint32_t m0 = ct * 32 + j, m1 = m0 + 32;
        const uint32_t last = g.M - 1;
        m0 = m0 < last ? m0 : last;
        m1 = m1 < last ? m1 : last;
        const uint32_t md = hh ? m1 : m0;
        if (WT == PPML_WTYPE_Q8_0R) {
            oq0 = m0 * nblk * 32u + hh * 16u;
            oq1 = m1 * nblk * 32u + hh * 16u;
            od = static_cast<uint32_t>(g.M) * nblk * 32u + md * nblk * 2u;
        } else if (WT == PPML_WTYPE_Q8_0) {
            oq0 = m0 * nblk * 34u + 2u + hh * 16u;
            oq1 = m1 * nblk * 34u + 2u + hh * 16u;
            od = md * nblk * 34u;
        } else {                                       // Q8_1: {half d; half s; int8 qs[32]}
            oq0 = m0 * nblk * 36u + 4u + hh * 16u;
            oq1 = m1 * nblk * 36u + 4u + hh * 16u;
            od = md * nblk * 36u;
        }
    }
    static __device__ __forceinline__ v4i load_q(const uint8_t* __restrict__ W, uint32_t off) {
        if (WT == PPML_WTYPE_Q8_0M) return *reinterpret_cast<const v4i*>(W + off);
        if (WT == PPML_WTYPE_Q8_0) {                   // 2-byte aligned records
            const uint16_t* q16 = reinterpret_cast<const uint16_t*>(W + off);
            v4i q;
#pragma unroll
            for (int c = 0; c < 4; ++c)
                q[c] = static_cast<int>(static_cast<uint32_t>(q16[2 * c]) | (static_cast<uint32_t>(q16[2 * c + 1]) << 16));
            return q;
        }
        typedef int v4i_u __attribute__((ext_vector_type(4), aligned(4)));
        return *reinterpret_cast<const v4i_u*>(W + off);
    }
    __device__ __forceinline__ void load(const uint8_t* __restrict__ W) {
        q0 = load_q(W, oq0);
        q1 = load_q(W, oq1);
        d_bits = *reinterpret_cast<const uint16_t*>(W + od);
    }
    __device__ __forceinline__ void advance() {
        oq0 += q_stride();
        oq1 += q_stride();
        od += d_stride();
    }
};

template <int NW, int P, int WT, bool DUMP>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(2))) void q8_linear_kernel(
    const uint8_t* __restrict__ W, const float* __restrict__ X, float* __restrict__ C,
    int M, int N, int nblk, int c_trans, int relu,
    uint8_t* __restrict__ xq_dump, int32_t* __restrict__ sums_dump) {
    static_assert(P % 2 == 0, "column tiles are processed in pairs");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int kc = nblk < KC_MAX ? nblk : KC_MAX;
    v4i* lds_a = reinterpret_cast<v4i*>(lds);                                        // [kc][64] fragments
    float* lds_d = reinterpret_cast<float*>(lds + static_cast<size_t>(kc) * 1024);   // [kc][32]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // uniform: keeps tile addressing scalar
    const int j = lane & 31;
    const int tok0 = blockIdx.x * TILE_TOK;
    const int K = nblk * QK;
    const int mct = (M + 31) / 32;
    const WGeom g{W, M, nblk, packed_tiles(M)};

    for (int ct_base = 0; ct_base < mct; ct_base += NW * P) {
        const int ct0 = ct_base + wave * P;
        v16f acc[P];
#pragma unroll
        for (int p = 0; p < P; ++p)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[p][r] = 0.0f;

        WPair<WT> wp[P / 2];
        if (ct0 < mct) {
#pragma unroll
            for (int pp = 0; pp < P / 2; ++pp) {
                wp[pp].init(g, ct0 + 2 * pp, lane);
                wp[pp].load(W);                        // block 0, in flight while X is quantized
            }
        }

        for (int b0 = 0; b0 < nblk; b0 += kc) {
            const int nb = (nblk - b0) < kc ? (nblk - b0) : kc;
            // ---------------- phase 1: quantize X[tok0..+32][b0*32 .. (b0+nb)*32) into LDS
            // (skipped when the whole K is already staged from an earlier column pass)
            if (ct_base == 0 || nblk > kc) {
                if (b0 > 0 || ct_base > 0) __syncthreads();        // previous readers are done
                const int units = nb * 4;                          // (8 rows) x (1 block) per wave step
                const int grp = lane >> 3, c8 = lane & 7;
                for (int u0 = wave; u0 < units; u0 += NW * UB) {
                    v4f xv[UB];
#pragma unroll
                    for (int s = 0; s < UB; ++s) {
                        int u = u0 + s * NW;
                        u = u < units ? u : units - 1;             // surplus slots repeat the last unit
                        const int row = (u & 3) * 8 + grp;
                        int tok = tok0 + row;
                        tok = tok < N ? tok : N - 1;               // rows past the end repeat the last row
                        xv[s] = *reinterpret_cast<const v4f_u*>(
                            X + static_cast<int64_t>(tok) * K + (b0 + (u >> 2)) * QK + c8 * 4);
                    }
#pragma unroll
                    for (int s = 0; s < UB; ++s) {
                        const int u = u0 + s * NW;
                        if (u >= units) break;                     // wave-uniform
                        const int row = (u & 3) * 8 + grp;
                        const int bl = u >> 2;
                        v4f x = xv[s];
                        if (relu) {
#pragma unroll
                            for (int c = 0; c < 4; ++c) x[c] = fmaxf(x[c], 0.0f);
                        }
                        const BlockQuant bq = quantize_block_lane(x);
                        // fragment order: block bl, k-half c8/4, row, dword c8%4
                        int* dst = reinterpret_cast<int*>(lds_a) + ((bl * 64 + (c8 >> 2) * 32 + row) * 4 + (c8 & 3));
                        *dst = static_cast<int>(bq.q4);
                        if (c8 == 0) lds_d[bl * 32 + row] = half_bits_to_float(bq.d_bits);
                        if (DUMP && xq_dump) {
                            const int tok = tok0 + row;
                            if (tok < N) {
                                uint8_t* blk = xq_dump + (static_cast<int64_t>(tok) * nblk + b0 + bl) * Q8_0_BYTES;
                                uint16_t* q16 = reinterpret_cast<uint16_t*>(blk + 2 + c8 * 4);
                                q16[0] = static_cast<uint16_t>(bq.q4 & 0xffffu);
                                q16[1] = static_cast<uint16_t>(bq.q4 >> 16);
                                if (c8 == 0) *reinterpret_cast<uint16_t*>(blk) = bq.d_bits;
                            }
                        }
                    }
                }
                __syncthreads();
            }

            // ---------------- phase 2: blocks ascending, P column tiles per wave, in pairs
            if (ct0 < mct) {
                for (int bl = 0; bl < nb; ++bl) {
                    const int b = b0 + bl;
                    const bool more = b + 1 < nblk;                                // last block: harmless re-read
                    const v4i afrag = lds_a[bl * 64 + lane];
                    const float da_lane = lds_d[bl * 32 + j];                      // rows of both scale blocks
#pragma unroll
                    for (int pp = 0; pp < P / 2; ++pp) {
                        v16i zero_i;
                        v32f zero_f;
#pragma unroll
                        for (int r = 0; r < 16; ++r) zero_i[r] = 0;
#pragma unroll
                        for (int r = 0; r < 32; ++r) zero_f[r] = 0.0f;
                        // rows = activation rows (A operand), columns = weight rows (B operand);
                        // the longest instruction goes first so the first settle can start earliest
                        const float dw_lane = half_bits_to_float(static_cast<uint16_t>(wp[pp].d_bits));
                        const v32f scale = __builtin_amdgcn_mfma_f32_32x32x1f32(da_lane, dw_lane, zero_f, 0, 0, 0);
                        const v16i sum0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(afrag, wp[pp].q0, zero_i, 0, 0, 0);
                        const v16i sum1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(afrag, wp[pp].q1, zero_i, 0, 0, 0);
                        // request block b+1 now that the MFMAs have read block b; it lands during the settle
                        __builtin_amdgcn_sched_barrier(0);
                        if (more) wp[pp].advance();
                        wp[pp].load(W);
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            acc[2 * pp][r] = __builtin_fmaf(static_cast<float>(sum0[r]), scale[r], acc[2 * pp][r]);
                            acc[2 * pp + 1][r] = __builtin_fmaf(static_cast<float>(sum1[r]), scale[16 + r], acc[2 * pp + 1][r]);
                        }
                        if (DUMP && sums_dump) {
#pragma unroll
                            for (int r = 0; r < 16; ++r) {
                                const int tok = tok0 + mfma32_row(r, lane);
                                const int m0 = (ct0 + 2 * pp) * 32 + j;
                                if (tok < N && m0 < M)
                                    sums_dump[(static_cast<int64_t>(tok) * M + m0) * nblk + b] = sum0[r];
                                if (tok < N && m0 + 32 < M)
                                    sums_dump[(static_cast<int64_t>(tok) * M + m0 + 32) * nblk + b] = sum1[r];
                            }
                        }
                    }
                }
            }
        }

        // ---------------- phase 3: store
        if (ct0 < mct) {
            const bool full = (tok0 + TILE_TOK <= N) && (c_trans != 0);
            if (full) {
                float* crow = C + static_cast<int64_t>(tok0 + 4 * (lane >> 5)) * M + ct0 * 32 + j;
#pragma unroll
                for (int p = 0; p < P; ++p) {
                    if ((ct0 + p) * 32 + j < M) {
#pragma unroll
                        for (int r = 0; r < 16; ++r)
                            __builtin_nontemporal_store(acc[p][r], crow + static_cast<int64_t>(8 * (r >> 2) + (r & 3)) * M + p * 32);
                    }
                }
            } else {
#pragma unroll
                for (int p = 0; p < P; ++p) {
                    const int m = (ct0 + p) * 32 + j;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int tok = tok0 + mfma32_row(r, lane);
                        if (tok < N && m < M) {
                            if (c_trans) C[static_cast<int64_t>(tok) * M + m] = acc[p][r];
                            else         C[static_cast<int64_t>(m) * N + tok] = acc[p][r];
                        }
                    }
                }
            }
        }
    }
}

template <int NW, int P, int WT>
int launch_q8_linear(const void* W, const float* X, float* C, int M, int N, int nblk, int c_trans,
                     int relu, void* xq_dump, int32_t* sums_dump, hipStream_t stream) {
    const int kc = nblk < KC_MAX ? nblk : KC_MAX;
    const size_t lds = static_cast<size_t>(kc) * (1024 + 32 * sizeof(float));
    const dim3 grid((N + TILE_TOK - 1) / TILE_TOK), block(NW * 64);
    if (xq_dump || sums_dump)
        hipLaunchKernelGGL((q8_linear_kernel<NW, P, WT, true>), grid, block, lds, stream,
                           static_cast<const uint8_t*>(W), X, C, M, N, nblk, c_trans, relu,
                           static_cast<uint8_t*>(xq_dump), sums_dump);
    else
        hipLaunchKernelGGL((q8_linear_kernel<NW, P, WT, false>), grid, block, lds, stream,
                           static_cast<const uint8_t*>(W), X, C, M, N, nblk, c_trans, relu,
                           static_cast<uint8_t*>(nullptr), static_cast<int32_t*>(nullptr));
    return check_launch("q8_linear_kernel");
}

template <int WT>
int dispatch_q8_linear(const void* W, const float* X, float* C, int M, int N, int nblk, int c_trans,
                       int relu, void* xq_dump, int32_t* sums_dump, hipStream_t stream) {
    const int mct = (M + 31) / 32;
    // waves split the output columns; pick the shape with the fewest idle column tiles
    if (mct <= 4)  return launch_q8_linear<2, 2, WT>(W, X, C, M, N, nblk, c_trans, relu, xq_dump, sums_dump, stream);
    if (mct <= 8)  return launch_q8_linear<4, 2, WT>(W, X, C, M, N, nblk, c_trans, relu, xq_dump, sums_dump, stream);
    if (mct <= 16) return launch_q8_linear<4, 4, WT>(W, X, C, M, N, nblk, c_trans, relu, xq_dump, sums_dump, stream);
    return launch_q8_linear<4, 6, WT>(W, X, C, M, N, nblk, c_trans, relu, xq_dump, sums_dump, stream);
}

}  // namespace
}  // namespace ppmlhip

using namespace ppmlhip;

extern "C" int quantize_rows_q8_0_hip(const float* x, void* y, int64_t ne, ppml_hip_stream_t stream) {
    if (!x || !y || ne <= 0 || (ne % QK) != 0) { set_error("quantize_rows_q8_0_hip: bad arguments (ne=%lld)", (long long)ne); return RC_BAD_ARGS; }
    const int64_t nblocks = ne / QK;
    const int64_t threads = nblocks * 8;
    const unsigned grid = static_cast<unsigned>((threads + 255) / 256);
    hipLaunchKernelGGL(quantize_rows_q8_0_kernel, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream),
                       x, static_cast<uint8_t*>(y), nblocks);
    return check_launch("quantize_rows_q8_0_kernel") ? RC_BAD_ARGS : RC_OK;   // reference launcher: 0 / 1
}

extern "C" int dequantize_q8_0_hip(const void* x, float* y, int64_t ne, ppml_hip_stream_t stream) {
    if (!x || !y || ne <= 0) { set_error("dequantize_q8_0_hip: bad arguments"); return RC_BAD_ARGS; }
    const unsigned grid = static_cast<unsigned>((ne + 255) / 256);
    hipLaunchKernelGGL(dequantize_q8_0_kernel, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint8_t*>(x), y, ne);
    return check_launch("dequantize_q8_0_kernel") ? RC_BAD_ARGS : RC_OK;
}

extern "C" size_t q8_weight_packed_bytes_hip(int M, int K) {
    if (M <= 0 || K <= 0 || (K % QK) != 0) return 0;
    const size_t tiles = static_cast<size_t>(packed_tiles(M));
    return tiles * static_cast<size_t>(K / QK) * (1024 + 32 * sizeof(uint16_t));
}

extern "C" int q8_weight_pack_hip(const void* W, int wtype, int M, int K, void* packed, ppml_hip_stream_t stream) {
    if (!W || !packed || M <= 0 || K <= 0) { set_error("q8_weight_pack_hip: bad arguments"); return RC_BAD_ARGS; }
    if ((K % QK) != 0) { set_error("q8_weight_pack_hip: K=%d is not a multiple of 32", K); return RC_K_NOT_32; }
    const int nblk = K / QK, mct = packed_tiles(M);
    const dim3 grid(mct * nblk), block(64);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint8_t* w = static_cast<const uint8_t*>(W);
    uint8_t* o = static_cast<uint8_t*>(packed);
    switch (wtype) {
        case PPML_WTYPE_Q8_0:  hipLaunchKernelGGL((q8_weight_pack_kernel<PPML_WTYPE_Q8_0>),  grid, block, 0, s, w, o, M, nblk, mct); break;
        case PPML_WTYPE_Q8_1:  hipLaunchKernelGGL((q8_weight_pack_kernel<PPML_WTYPE_Q8_1>),  grid, block, 0, s, w, o, M, nblk, mct); break;
        case PPML_WTYPE_Q8_0R: hipLaunchKernelGGL((q8_weight_pack_kernel<PPML_WTYPE_Q8_0R>), grid, block, 0, s, w, o, M, nblk, mct); break;
        default: set_error("q8_weight_pack_hip: unsupported source wtype %d", wtype); return RC_WTYPE;
    }
    return check_launch("q8_weight_pack_kernel");
}

extern "C" int mul_mat_q8_ex_hip(const void* W, const float* X, float* C, int M, int N, int K, int wtype,
                                 int c_trans, int flags, void* xq_dump, int32_t* sums_dump,
                                 ppml_hip_stream_t stream) {
    if (!W || !X || !C || M <= 0 || N <= 0 || K <= 0) { set_error("mul_mat_q8_hip: bad arguments (M=%d N=%d K=%d)", M, N, K); return RC_BAD_ARGS; }
    if ((K % QK) != 0) { set_error("mul_mat_q8_hip: K=%d is not a multiple of 32", K); return RC_K_NOT_32; }
    const int nblk = K / QK;
    const int relu = flags & 1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    stats_record(M, K, N);
    switch (wtype) {
        case PPML_WTYPE_Q8_0:  return dispatch_q8_linear<PPML_WTYPE_Q8_0>(W, X, C, M, N, nblk, c_trans, relu, xq_dump, sums_dump, s);
        case PPML_WTYPE_Q8_1:  return dispatch_q8_linear<PPML_WTYPE_Q8_1>(W, X, C, M, N, nblk, c_trans, relu, xq_dump, sums_dump, s);
        case PPML_WTYPE_Q8_0R: return dispatch_q8_linear<PPML_WTYPE_Q8_0R>(W, X, C, M, N, nblk, c_trans, relu, xq_dump, sums_dump, s);
        case PPML_WTYPE_Q8_0M: return dispatch_q8_linear<PPML_WTYPE_Q8_0M>(W, X, C, M, N, nblk, c_trans, relu, xq_dump, sums_dump, s);
        default: set_error("mul_mat_q8_hip: unsupported wtype %d", wtype); return RC_WTYPE;
    }
}

extern "C" int mul_mat_q8_hip(const void* W, const float* X, float* C, int M, int N, int K, int wtype,
                              int c_trans, int* path_out, ppml_hip_stream_t stream) {
    if (path_out) *path_out = 0;
    const int rc = mul_mat_q8_ex_hip(W, X, C, M, N, K, wtype, c_trans, 0, nullptr, nullptr, stream);
    if (rc == RC_OK && path_out) *path_out = 1;
    return rc;
}
