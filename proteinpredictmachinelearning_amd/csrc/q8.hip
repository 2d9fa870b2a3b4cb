// Q8_0 path for gfx950: row quantizer, dequantizer, weight repack and the fused
// quantize + int8-MFMA linear kernel.
//
// Reference behaviour restated here (paths relative to the reference tree):
//   quantizer arithmetic     include/ppml/QuantBlocks.h:62-79
//   block dot and settlement src/cuda/MulMatQ8Kernel.cu:120-142
//   launcher contract        src/cuda/MulMatQ8Kernel.cu:476-547, src/cuda/QuantKernels.cu:86-109
#include "common.hpp"
#include <type_traits>
#include <cstdlib>
#include <mutex>
#include <cstring>

namespace ppmlhip {
namespace {

// ------------------------------------------------------------------------------------------
// Quantizer arithmetic shared by the standalone and the fused kernel.
// ------------------------------------------------------------------------------------------

// max over each aligned group of 4 lanes (one Q8 block when every lane holds 8 elements) of a value that is
// not negative and not NaN: such floats order like their bit patterns, and an integer max has no signalling
// NaN to quiet, so each step is a single v_max_u32 that takes its other operand through DPP
__device__ __forceinline__ float group4_max(float v) {
    uint32_t b = __float_as_uint(v) & 0x7fffffffu;     // (a maximum of +0 and -0 may come out as -0: not the largest pattern)
    uint32_t o;
    o = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(b), 0xB1, 0xf, 0xf, false));  // lane ^ 1
    b = b > o ? b : o;
    o = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(b), 0x4E, 0xf, 0xf, false));  // lane ^ 2
    b = b > o ? b : o;
    return __uint_as_float(b);
}

struct BlockQuant {
    uint32_t q_lo, q_hi;  // this lane's 8 quants, element c in byte c % 4 of word c / 4
    uint16_t d_bits;      // fp16 scale of the block
    float d;              // the same scale before rounding to half
};

// round(t) for |t| <= 200 as one add and one truncating convert: adding the largest float below
// one half (with t's sign) carries exactly the ties and nothing else over the integer boundary,
// so the result equals (int)roundf(t) -- half away from zero -- for every binary32 t in range
// (checked exhaustively against roundf on the host).
__device__ __forceinline__ int round_half_away_to_int(float t) {
    const float h = __int_as_float((__float_as_int(t) & 0x80000000) | 0x3effffff);
    return static_cast<int>(t + h);
}

__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d) {
    const uint32_t ab = __builtin_amdgcn_perm(static_cast<uint32_t>(b), static_cast<uint32_t>(a), 0x0c0c0400u);
    const uint32_t cd = __builtin_amdgcn_perm(static_cast<uint32_t>(d), static_cast<uint32_t>(c), 0x0c0c0400u);
    return __builtin_amdgcn_perm(cd, ab, 0x05040100u);
}

// (|v|, v) of the first element of the block that reaches the block's largest magnitude, combined
// over an aligned group of 4 lanes that hold the block in element order: on equal magnitudes the
// lower lane wins, as the sequential scan with a strict `>` does (include/ppml/QuantBlocks.h:86-90).
__device__ __forceinline__ void group4_first_max(float& a, float& v) {
    const int lane = static_cast<int>(__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)));
    {
        const float oa = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(a), 0xB1, 0xf, 0xf, false));
        const float ov = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, false));
        const bool low = (lane & 1) == 0;              // this lane is the lower one of the pair
        const bool keep = low ? (a >= oa) : (a > oa);
        v = keep ? v : ov;
        a = keep ? a : oa;
    }
    {
        const float oa = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(a), 0x4E, 0xf, 0xf, false));
        const float ov = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, false));
        const bool low = (lane & 2) == 0;
        const bool keep = low ? (a >= oa) : (a > oa);
        v = keep ? v : ov;
        a = keep ? a : oa;
    }
}

// amax / 127 in three operations: q0 = a * c with c = RN(1 / 127), the exact remainder r = a - 127 q0 from one
// fma, q0 + r * c.  Equal to the IEEE quotient for every finite a >= 0, subnormals included (all 2^31 - 2^23
// values compared on the device); a = +inf gives NaN here and takes the caller's slow path.
__device__ __forceinline__ float div_by_127(float a) {
    const float c = 0x1.020408p-7f;
    const float q0 = a * c;
    const float r = __builtin_fmaf(-127.0f, q0, a);
    return __builtin_fmaf(r, c, q0);
}

// 1 / d in three operations: the hardware's approximation and one Newton step.  Equal to the IEEE reciprocal
// whenever d and 1 / d are both normal numbers, 2^-126 <= |d| <= 2^126 (all values compared on the device;
// outside that range the step's own arithmetic underflows).
__device__ __forceinline__ float rcp_normal(float d) {
    const float y0 = __builtin_amdgcn_rcpf(d);
    const float e = __builtin_fmaf(-d, y0, 1.0f);
    return __builtin_fmaf(e, y0, y0);
}
__device__ __forceinline__ bool rcp_normal_ok(float d) {
    return ((__float_as_uint(d) & 0x7fffffffu) - 0x00800000u) <= (0x7e800000u - 0x00800000u);
}

// x0,x1 hold elements 8*c4 .. 8*c4+7 of one 32-element block, the 4 lanes of an aligned group hold
// the whole block.  IEEE division for the scale and its reciprocal, round half away from zero.
//   Q81 = false: d = amax / 127, clamp to +-127             (include/ppml/QuantBlocks.h:62-79)
//   Q81 = true : d = vmax / -128 with vmax the signed element of largest magnitude, clamp to
//                [-128, 127]; *qsum receives this lane's share of the sum of the quants
//                                                            (include/ppml/QuantBlocks.h:81-111)
//   RELU       : the block is max(x, 0).  Nothing is spent on forming it: its largest magnitude is the
//                signed maximum of x and zero, and the quants of its zeros are made zero by the clamp
//                (x < 0 lands on the side of zero opposite to the kept elements; NaN converts to 0 either
//                way, like the 0 that max(NaN, 0) is).
// The two divisions take the short forms above whenever every block of the wave is in their proven range
// (an all-zero block counts: its reciprocal is replaced by 0 below), else the compiler's IEEE expansion.
template <bool Q81, bool RELU = false>
__device__ __forceinline__ BlockQuant quantize_block_lane(v4f x0, v4f x1, int* qsum = nullptr) {
    float amax = 0.0f, vmax = 0.0f;
    if (RELU) {
#pragma unroll
        for (int c = 0; c < 4; ++c) amax = fmaxf(amax, x0[c]);          // fmaxf drops NaN like std::fmax
#pragma unroll
        for (int c = 0; c < 4; ++c) amax = fmaxf(amax, x1[c]);
        amax = group4_max(amax);
        vmax = amax;
    } else if (Q81) {
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const float x = c < 4 ? x0[c & 3] : x1[c & 3];
            const bool gt = fabsf(x) > amax;            // false for NaN: ignored like the host's scan
            vmax = gt ? x : vmax;
            amax = gt ? fabsf(x) : amax;
        }
        group4_first_max(amax, vmax);
    } else {
#pragma unroll
        for (int c = 0; c < 4; ++c) amax = fmaxf(amax, fabsf(x0[c]));   // fmaxf drops NaN like std::fmax
#pragma unroll
        for (int c = 0; c < 4; ++c) amax = fmaxf(amax, fabsf(x1[c]));
        amax = group4_max(amax);
    }
    float d = Q81 ? vmax * -0x1p-7f : div_by_127(amax);                // the division by -128 is an exact scaling, or a subnormal rounded once either way
    float inv;
    const bool zero = amax == 0.0f;
    const bool fast = __builtin_amdgcn_ballot_w64(!(zero || rcp_normal_ok(d))) == 0;   // wave-uniform
    if (__builtin_expect(fast, 1)) {
        inv = rcp_normal(d);
    } else {
        d = Q81 ? vmax / -128.0f : amax / 127.0f;
        inv = 1.0f / d;
    }
    if (Q81) {
        if (zero) d = 0.0f;
        if (d == 0.0f) inv = 0.0f;
    } else if (zero) {
        inv = 0.0f;
    }
    BlockQuant out;
    out.d_bits = __half_as_ushort(__float2half_rn(d));
    out.d = d;
    int q[8];
    constexpr int QMIN = Q81 ? -128 : (RELU ? 0 : -127);
    constexpr int QMAX = (Q81 && RELU) ? 0 : 127;
    if (!Q81 && fast) {
        // With d and 1 / d normal, |x * inv| <= 127 (1 + 2^-23)(1 + 2^-24) for every element of the block, which
        // rounds to at most 127: the clamp has nothing to do.  Under RELU the kept elements are positive, so the
        // rounding offset needs no sign, and the unsigned conversion turns the others (and NaN) into the 0 they are.
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const float t = (c < 4 ? x0[c & 3] : x1[c & 3]) * inv;
            if (RELU) {
                const float u = t + 0x1.fffffep-2f;
                unsigned qu;
                asm("v_cvt_u32_f32 %0, %1" : "=v"(qu) : "v"(u));
                q[c] = static_cast<int>(qu);
            } else {
                q[c] = round_half_away_to_int(t);
            }
        }
    } else {
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            q[c] = round_half_away_to_int((c < 4 ? x0[c & 3] : x1[c & 3]) * inv);
            q[c] = q[c] > QMAX ? QMAX : (q[c] < QMIN ? QMIN : q[c]);
        }
    }
    if (Q81 && qsum) *qsum = q[0] + q[1] + q[2] + q[3] + q[4] + q[5] + q[6] + q[7];
    out.q_lo = pack4(q[0], q[1], q[2], q[3]);
    out.q_hi = pack4(q[4], q[5], q[6], q[7]);
    return out;
}

__device__ __forceinline__ float half_bits_to_float(uint16_t h) {
    return __half2float(__ushort_as_half(h));
}

// 8 quants of block `blk` (2-byte aligned 34-byte record) written by the lane that owns them
__device__ __forceinline__ void store_block_part(uint8_t* blk, int c4, const BlockQuant& bq) {
    uint16_t* q16 = reinterpret_cast<uint16_t*>(blk + 2 + c4 * 8);
    q16[0] = static_cast<uint16_t>(bq.q_lo & 0xffffu);
    q16[1] = static_cast<uint16_t>(bq.q_lo >> 16);
    q16[2] = static_cast<uint16_t>(bq.q_hi & 0xffffu);
    q16[3] = static_cast<uint16_t>(bq.q_hi >> 16);
    if (c4 == 0) *reinterpret_cast<uint16_t*>(blk) = bq.d_bits;
}

// ------------------------------------------------------------------------------------------
// Standalone row quantizer / dequantizer (interleaved 34-byte blocks in HBM)
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void quantize_rows_q8_0_kernel(const float* __restrict__ x,
                                                                 uint8_t* __restrict__ y,
                                                                 int64_t nblocks) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    int64_t ib = t >> 2;
    const int c4 = static_cast<int>(t & 3);
    const bool live = ib < nblocks;
    if (!live) ib = nblocks - 1;                       // keep the whole 4-lane group convergent
    const float* src = x + ib * QK + c4 * 8;
    const v4f x0 = *reinterpret_cast<const v4f_u*>(src);
    const v4f x1 = *reinterpret_cast<const v4f_u*>(src + 4);
    const BlockQuant bq = quantize_block_lane<false>(x0, x1);
    if (!live) return;
    store_block_part(y + ib * Q8_0_BYTES, c4, bq);
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

// Q8_1 records {half d, half s, int8 qs[32]} (include/ppml/QuantBlocks.h:38-41), s = d * sum(qs)
__global__ __launch_bounds__(256) void quantize_rows_q8_1_kernel(const float* __restrict__ x,
                                                                 uint8_t* __restrict__ y,
                                                                 int64_t nblocks) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    int64_t ib = t >> 2;
    const int c4 = static_cast<int>(t & 3);
    const bool live = ib < nblocks;
    if (!live) ib = nblocks - 1;                       // keep the whole 4-lane group convergent
    const float* src = x + ib * QK + c4 * 8;
    const v4f x0 = *reinterpret_cast<const v4f_u*>(src);
    const v4f x1 = *reinterpret_cast<const v4f_u*>(src + 4);
    int qsum = 0;
    const BlockQuant bq = quantize_block_lane<true>(x0, x1, &qsum);
    qsum += __builtin_amdgcn_update_dpp(0, qsum, 0xB1, 0xf, 0xf, false);   // lane ^ 1
    qsum += __builtin_amdgcn_update_dpp(0, qsum, 0x4E, 0xf, 0xf, false);   // lane ^ 2
    if (!live) return;
    uint8_t* blk = y + ib * Q8_1_BYTES;
    uint32_t* q32 = reinterpret_cast<uint32_t*>(blk + 4 + c4 * 8);       // records are 4-byte aligned
    q32[0] = bq.q_lo;
    q32[1] = bq.q_hi;
    if (c4 == 0) {
        // s is made from the fp32 scale, like the reference: d * float(sum), then one rounding to half
        reinterpret_cast<uint16_t*>(blk)[0] = bq.d_bits;
        reinterpret_cast<uint16_t*>(blk)[1] = __half_as_ushort(__float2half_rn(bq.d * static_cast<float>(qsum)));
    }
}

__global__ __launch_bounds__(256) void dequantize_q8_1_kernel(const uint8_t* __restrict__ x,
                                                              float* __restrict__ y, int64_t ne) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= ne) return;
    const int64_t ib = i / QK;
    const int iq = static_cast<int>(i - ib * QK);
    const uint8_t* blk = x + ib * Q8_1_BYTES;
    const float d = half_bits_to_float(*reinterpret_cast<const uint16_t*>(blk));
    y[i] = d * static_cast<float>(static_cast<int8_t>(blk[4 + iq]));
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
//   phase 1  the work-group streams its 32 x K slice of X once from HBM (16-byte loads, 4 lanes
//            per Q8 block, block absmax by DPP), quantizes it and leaves it in LDS already in
//            MFMA-fragment order, scales beside it as f32.  Nothing quantized goes back to HBM.
//   phase 2  the waves share out the output columns in pairs of 32-column tiles.  For one pair a
//            wave walks the blocks in ascending order; per block it issues two
//            v_mfma_i32_32x32x32_i8 -> exact int32 block sums, and one v_mfma_f32_32x32x1_2b_f32
//            whose two 32x32 outer products are the scale products d_w[col]*d_a[row] of both tiles
//            (each the exact product of two halves), then settles
//            acc = fma(float(sumi), d_w*d_a, acc) on the VALU.  The weight fragments of the next
//            block are requested as soon as the MFMAs of this one have read theirs.
//   phase 3  the pair is stored at once (16 bytes per lane), so the output streams to HBM while the
//            other pairs are still being computed; only 32 accumulator registers are ever live,
//            which lets four work-groups share a CU.
//
// MFMA roles: A = weight rows (output rows of the instruction), B = activation rows (output
// columns), so a lane ends up with 4 consecutive output features of one token per register quad.
//
// LDS per work-group: kc * 1152 bytes, kc = blocks of K staged at once (at most KC_MAX).  For longer
// rows K is walked in chunks and the partial result of every output is carried in C itself, which
// keeps the per-output block order intact.
// ------------------------------------------------------------------------------------------

constexpr int TILE_TOK = 32;
// Cache policy of the output stores of the weight-stationary kernel: sc0 | nt.  The output is
// written once and not read again by this kernel; streaming stores measured 15 % faster end to
// end than default ones at the MSA QKV shape (the same hint on the activation loads costs 4 %).
constexpr int WS_STORE_AUX = 3;
constexpr int WS_MAGIC_BITS = 0x4B400000;   // binary32 1.5 * 2^23: accumulator start of the int8 MFMAs whose sums are read as floats
constexpr int WS_NBUF = 3;          // quantized activation tiles the weight-stationary kernel keeps in LDS
constexpr int KC_MAX = 56;          // blocks of K staged in LDS at once (63 KiB)
constexpr int UB = 4;               // quantizer units (8 rows x 2 blocks) a wave keeps in flight

typedef float v32f __attribute__((ext_vector_type(32)));

// Read cursor over the weight data of one pair of column tiles (ct, ct+1): 32-bit byte offsets
// from the weight base, advanced by a fixed stride per Q8 block.
template <int WT>
struct WPair {
    uint32_t oq0, oq1, od;   // offsets of this lane's fragment of tile ct, of tile ct+1, and of its scale
    v4i q0, q1;              // fragments of the current block
    uint32_t d_bits;         // fp16 scale of tile ct (lanes 0-31) / ct+1 (lanes 32-63); converted at use

    static constexpr uint32_t q_stride() {
        return WT == PPML_WTYPE_Q8_0M ? 1024u : WT == PPML_WTYPE_Q8_0R ? 32u : WT == PPML_WTYPE_Q8_0 ? 34u : 36u;
    }
    static constexpr uint32_t d_stride() {
        return WT == PPML_WTYPE_Q8_0M ? 64u : WT == PPML_WTYPE_Q8_0R ? 2u : WT == PPML_WTYPE_Q8_0 ? 34u : 36u;
    }
    // cursor at block b of the pair starting at tile ct
    __device__ __forceinline__ void init(const WGeom& g, int ct, int b, int lane) {
        const uint32_t j = lane & 31, hh = lane >> 5;
        const uint32_t nblk = g.nblk;
        if (WT == PPML_WTYPE_Q8_0M) {
            // pairs past the end repeat the last pair; their results are never stored
            const uint32_t c = ct + 1 < g.mct_pad ? ct : g.mct_pad - 2;
            oq0 = ((c * nblk + b) * 64u + lane) * 16u;
            oq1 = oq0 + nblk * 1024u;
            od = static_cast<uint32_t>(g.mct_pad) * nblk * 1024u + (((c + hh) * nblk + b) * 32u + j) * 2u;
            return;
        }
        // rows past the end repeat the last row; their results are never stored
        uint32_t m0 = ct * 32 + j, m1 = m0 + 32;
        const uint32_t last = g.M - 1;
        m0 = m0 < last ? m0 : last;
        m1 = m1 < last ? m1 : last;
        const uint32_t md = hh ? m1 : m0;
        if (WT == PPML_WTYPE_Q8_0R) {
            oq0 = (m0 * nblk + b) * 32u + hh * 16u;
            oq1 = (m1 * nblk + b) * 32u + hh * 16u;
            od = static_cast<uint32_t>(g.M) * nblk * 32u + (md * nblk + b) * 2u;
        } else if (WT == PPML_WTYPE_Q8_0) {
            oq0 = (m0 * nblk + b) * 34u + 2u + hh * 16u;
            oq1 = (m1 * nblk + b) * 34u + 2u + hh * 16u;
            od = (md * nblk + b) * 34u;
        } else {                                       // Q8_1: {half d; half s; int8 qs[32]}
            oq0 = (m0 * nblk + b) * 36u + 4u + hh * 16u;
            oq1 = (m1 * nblk + b) * 36u + 4u + hh * 16u;
            od = (md * nblk + b) * 36u;
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

// address of C(tok, m) and whether a lane may touch it
struct COut {
    float* C;
    int M, N, c_trans;
    __device__ __forceinline__ float* at(int tok, int m) const {
        return c_trans ? C + static_cast<int64_t>(tok) * M + m : C + static_cast<int64_t>(m) * N + tok;
    }
};

template <int NW, int WT, bool DUMP>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(4, 4))) void q8_linear_kernel(
    const uint8_t* __restrict__ W, const float* __restrict__ X, float* __restrict__ C,
    int M, int N, int nblk, int kc, int c_trans, int relu,
    uint8_t* __restrict__ xq_dump, int32_t* __restrict__ sums_dump) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    v4i* lds_a = reinterpret_cast<v4i*>(lds);                                        // [kc][64] fragments
    float* lds_d = reinterpret_cast<float*>(lds + static_cast<size_t>(kc) * 1024);   // [kc][32]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // uniform: keeps tile addressing scalar
    const int j = lane & 31, hh = lane >> 5;
    const int tok0 = blockIdx.x * TILE_TOK;
    const int K = nblk * QK;
    const int npairs = (M + 63) / 64;
    const WGeom g{W, M, nblk, packed_tiles(M)};
    const COut out{C, M, N, c_trans};
    const int tok = tok0 + j;                          // this lane's activation row in every MFMA result

    for (int b0 = 0; b0 < nblk; b0 += kc) {
        const int nb = (nblk - b0) < kc ? (nblk - b0) : kc;
        // ---------------- phase 1: quantize X[tok0..+32][b0*32 .. (b0+nb)*32) into LDS
        if (b0 > 0) __syncthreads();                   // readers of the previous chunk are done
        WPair<WT> wp;
        {
            const int npair_b = (nb + 1) >> 1;
            const int units = npair_b * 4;             // (8 rows) x (2 blocks) per wave step
            const int grp = lane >> 2, c4 = lane & 3;
            const int urow = grp & 7, ublk = grp >> 3; // row and block within the unit
            for (int u0 = wave; u0 < units; u0 += NW * UB) {
                v4f xv[UB][2];
#pragma unroll
                for (int s = 0; s < UB; ++s) {
                    int u = u0 + s * NW;
                    u = u < units ? u : units - 1;     // surplus slots repeat the last unit
                    int bl = (u >> 2) * 2 + ublk;
                    bl = bl < nb ? bl : nb - 1;        // odd block count: repeat the last block
                    int t = tok0 + (u & 3) * 8 + urow;
                    t = t < N ? t : N - 1;             // rows past the end repeat the last row
                    const float* src = X + static_cast<int64_t>(t) * K + (b0 + bl) * QK + c4 * 8;
                    xv[s][0] = *reinterpret_cast<const v4f_u*>(src);
                    xv[s][1] = *reinterpret_cast<const v4f_u*>(src + 4);
                }
                if (u0 == wave && wave < npairs) {
                    // first weight block of this wave's first pair: requested behind the activation
                    // loads, lands while they are being quantized
                    wp.init(g, 2 * wave, b0, lane);
                    wp.load(W);
                }
#pragma unroll
                for (int s = 0; s < UB; ++s) {
                    const int u = u0 + s * NW;
                    if (u >= units) break;             // wave-uniform
                    const int row = (u & 3) * 8 + urow;
                    const int bl = (u >> 2) * 2 + ublk;
                    const v4f x0 = xv[s][0], x1 = xv[s][1];
                    const BlockQuant bq = (relu & 2) ? ((relu & 1) ? quantize_block_lane<true, true>(x0, x1) : quantize_block_lane<true, false>(x0, x1))
                                                     : ((relu & 1) ? quantize_block_lane<false, true>(x0, x1) : quantize_block_lane<false, false>(x0, x1));
                    if (bl < nb) {
                        // fragment order: block bl, k-half c4/2, row, dword pair c4%2
                        uint2* dst = reinterpret_cast<uint2*>(lds_a) + ((bl * 64 + (c4 >> 1) * 32 + row) * 2 + (c4 & 1));
                        *dst = uint2{bq.q_lo, bq.q_hi};
                        if (c4 == 0) lds_d[bl * 32 + row] = half_bits_to_float(bq.d_bits);
                        if (DUMP && xq_dump) {
                            const int t = tok0 + row;
                            if (t < N)
                                store_block_part(xq_dump + (static_cast<int64_t>(t) * nblk + b0 + bl) * Q8_0_BYTES, c4, bq);
                        }
                    }
                }
            }
            if (units <= wave && wave < npairs) {      // this wave had nothing to quantize
                wp.init(g, 2 * wave, b0, lane);
                wp.load(W);
            }
        }
        __syncthreads();

        // ---------------- phase 2 + 3: one pair of column tiles at a time
        for (int pr = wave; pr < npairs; pr += NW) {
            const int ct = 2 * pr;
            v16f acc0, acc1;
            if (b0 == 0) {
#pragma unroll
                for (int r = 0; r < 16; ++r) { acc0[r] = 0.0f; acc1[r] = 0.0f; }
            } else {
                // later chunk of a long row: the running sums were parked in C
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m = ct * 32 + mfma32_row(r, lane);
                    acc0[r] = (tok < N && m < M) ? *out.at(tok, m) : 0.0f;
                    acc1[r] = (tok < N && m + 32 < M) ? *out.at(tok, m + 32) : 0.0f;
                }
            }
            for (int bl = 0; bl < nb; ++bl) {
                const v4i afrag = lds_a[bl * 64 + lane];
                const float da_lane = lds_d[bl * 32 + j];                  // columns of both scale blocks
                v16i zero_i;
                v32f zero_f;
#pragma unroll
                for (int r = 0; r < 16; ++r) zero_i[r] = 0;
#pragma unroll
                for (int r = 0; r < 32; ++r) zero_f[r] = 0.0f;
                // the longest instruction goes first so the first settle can start earliest
                const float dw_lane = half_bits_to_float(static_cast<uint16_t>(wp.d_bits));
                const v32f scale = __builtin_amdgcn_mfma_f32_32x32x1f32(dw_lane, da_lane, zero_f, 0, 0, 0);
                const v16i sum0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(wp.q0, afrag, zero_i, 0, 0, 0);
                const v16i sum1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(wp.q1, afrag, zero_i, 0, 0, 0);
                // request the next block (or the first block of this wave's next pair) now that the
                // MFMAs have read this one; it lands during the settle
                __builtin_amdgcn_sched_barrier(0);
                if (bl + 1 < nb) wp.advance();
                else if (pr + NW < npairs) wp.init(g, ct + 2 * NW, b0, lane);
                wp.load(W);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    acc0[r] = __builtin_fmaf(static_cast<float>(sum0[r]), scale[r], acc0[r]);
                    acc1[r] = __builtin_fmaf(static_cast<float>(sum1[r]), scale[16 + r], acc1[r]);
                }
                if (DUMP && sums_dump) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int m = ct * 32 + mfma32_row(r, lane);
                        if (tok < N && m < M)
                            sums_dump[(static_cast<int64_t>(tok) * M + m) * nblk + b0 + bl] = sum0[r];
                        if (tok < N && m + 32 < M)
                            sums_dump[(static_cast<int64_t>(tok) * M + m + 32) * nblk + b0 + bl] = sum1[r];
                    }
                }
            }
            // ---------------- phase 3: store the pair
            if (tok < N) {
                if (c_trans) {
                    float* crow = C + static_cast<int64_t>(tok) * M + ct * 32 + 4 * hh;
#pragma unroll
                    for (int t = 0; t < 2; ++t) {
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const int m = (ct + t) * 32 + 8 * q + 4 * hh;
                            const v16f& a = t ? acc1 : acc0;
                            if (m + 3 < M) {
                                v4f v = {a[4 * q], a[4 * q + 1], a[4 * q + 2], a[4 * q + 3]};
                                *reinterpret_cast<v4f_u*>(crow + t * 32 + 8 * q) = v;
                            } else {
#pragma unroll
                                for (int c = 0; c < 4; ++c)
                                    if (m + c < M) crow[t * 32 + 8 * q + c] = a[4 * q + c];
                            }
                        }
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int m = ct * 32 + mfma32_row(r, lane);
                        if (m < M) C[static_cast<int64_t>(m) * N + tok] = acc0[r];
                        if (m + 32 < M) C[static_cast<int64_t>(m + 32) * N + tok] = acc1[r];
                    }
                }
            }
        }
    }
}

template <int NW, int WT>
int launch_q8_linear(const void* W, const float* X, float* C, int M, int N, int nblk, int c_trans,
                     int relu, void* xq_dump, int32_t* sums_dump, hipStream_t stream) {
    const int kc = nblk < KC_MAX ? nblk : KC_MAX;
    const size_t lds = static_cast<size_t>(kc) * (1024 + 32 * sizeof(float));
    const dim3 grid((N + TILE_TOK - 1) / TILE_TOK), block(NW * 64);
    if (xq_dump || sums_dump)
        hipLaunchKernelGGL((q8_linear_kernel<NW, WT, true>), grid, block, lds, stream,
                           static_cast<const uint8_t*>(W), X, C, M, N, nblk, kc, c_trans, relu,
                           static_cast<uint8_t*>(xq_dump), sums_dump);
    else
        hipLaunchKernelGGL((q8_linear_kernel<NW, WT, false>), grid, block, lds, stream,
                           static_cast<const uint8_t*>(W), X, C, M, N, nblk, kc, c_trans, relu,
                           static_cast<uint8_t*>(nullptr), static_cast<int32_t*>(nullptr));
    return check_launch("q8_linear_kernel");
}

// ------------------------------------------------------------------------------------------
// Weight-stationary form of the same linear, for Q8_0M weights small enough to live in registers
// (M*K up to 256 Ki elements: every projection the reference quantizes, src/model/PPML.cpp:4434-4437).
//
// One work-group of 8 waves per CU walks over token tiles.  Wave w keeps the fragments and scales
// of its TPW column tiles in VGPRs for the whole kernel, so the inner loop has no weight traffic at
// all and the only vector-memory operations are the activation loads and the output stores:
//
//   loads of tile i+1 are issued before the MFMA work of tile i and its stores, so waiting for
//   them never waits for a store (the VMEM counter retires in order), and the activation read,
//   the arithmetic and the output write of neighbouring tiles overlap inside one work-group.
//
// Per column tile the blocks are walked in ascending order.  Each step issues the two MFMAs of
// block b+1 -- v_mfma_i32_32x32x32_i8 for the exact block sums and v_mfma_f32_32x32x2_f32 for the
// 32x32 scale products d_a[row]*d_w[col] (second K slot zero) -- and then settles block b on the
// VALU, so the matrix pipe runs one block ahead of the VALU and neither waits for the other.  A
// tile is stored as soon as its last block is settled, under the arithmetic of the next tile.
// MFMA roles: A = activation rows, B = weight rows, so a store instruction writes two full
// 128-byte lines.  LDS holds three quantized tiles and a count of the waves that have written each,
// so the loop needs no barrier: waves drift apart by up to a third of a tile instead of meeting.
// ------------------------------------------------------------------------------------------
// A value the optimizer cannot see through (always 1).  Branching on it puts the guarded code in a
// basic block of its own: the fully unrolled MFMA steps below would otherwise all be issued up
// front, since nothing orders them, and their result registers would spill.
__device__ __forceinline__ int opaque_one() {
    int one = 1;
    asm volatile("" : "+s"(one));
    return one;
}

// VGPRs the compiler may allocate in the weight-stationary kernel; the ones above hold the
// activation tile in flight (see load_tile_async) and are touched by inline assembly only.
constexpr int ws_staging_regs(int nblk, int nw = 8) {   // 8 registers per unit of (8 rows x 2 blocks) a wave loads
    return (2 * nblk + nw - 1) / nw * 8 < 16 ? 16 : (2 * nblk + nw - 1) / nw * 8;
}
constexpr int ws_compiler_vgprs(int nblk, int nw = 8) { return 256 - ws_staging_regs(nblk, nw); }

template <int NW, int TPW, int NBLK, int WL, bool DUMP, bool Q81, bool CSPLIT, bool QEARLY, bool CT0>
__device__ __forceinline__ void q8_linear_ws_body(
    const uint8_t* __restrict__ W, const float* __restrict__ X, float* __restrict__ C,
    int M, int N, int ntiles, int npart, int relu,
    uint8_t* __restrict__ xq_dump, int32_t* __restrict__ sums_dump) {
    static_assert(NBLK % 2 == 0, "the quantizer stages blocks in pairs");
    constexpr int K = NBLK * QK;
    constexpr int NUNITS = 2 * NBLK;                   // (8 rows) x (2 blocks) each
    constexpr int UPW = (NUNITS + NW - 1) / NW;        // units per wave
    constexpr int STEPS = TPW * NBLK;
    // LDS: three quantized activation tiles (fragments + scales) and this work-group's weight scales.
    extern __shared__ __attribute__((aligned(16))) uint8_t ws_lds[];
    v4i (*lds_a)[NBLK * 64] = reinterpret_cast<v4i (*)[NBLK * 64]>(ws_lds);
    constexpr size_t OFF_D = static_cast<size_t>(WS_NBUF) * NBLK * 1024;
    constexpr size_t OFF_WD = OFF_D + static_cast<size_t>(WS_NBUF) * NBLK * 256;
    constexpr size_t OFF_READY = OFF_WD + static_cast<size_t>(NW) * TPW * NBLK * 256;
    constexpr size_t OFF_WQ = OFF_READY + 16;
    // activation scales [buffer][block][32 rows] and weight scales [wave][column tile][block][32 columns],
    // kept as the bits of the halves they are, each followed by three zero halves: an entry is a lane's
    // whole operand of the scale MFMA, and 64 consecutive entries serve one such MFMA over a pair of blocks
    uint2 (*lds_d)[NBLK * 32] = reinterpret_cast<uint2 (*)[NBLK * 32]>(ws_lds + OFF_D);
    uint2* lds_wd = reinterpret_cast<uint2*>(ws_lds + OFF_WD);
    // ready[b]: how many waves have written their share of the tile currently being put in buffer b
    // (counts up for the life of the kernel; the k-th filling of a buffer is complete at k * NW)
    unsigned* lds_ready = reinterpret_cast<unsigned*>(ws_lds + OFF_READY);
    // fragments of the last WL column tiles of every wave, when the register file cannot hold all TPW
    v4i* lds_wq = reinterpret_cast<v4i*>(ws_lds + OFF_WQ);   // [NW][WL][NBLK][64]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 31, hh = lane >> 5;
    const int mct_pad = packed_tiles(M);
    const int grp = lane >> 2, c4 = lane & 3;
    const int urow = grp & 7, ublk = grp >> 3;
    const __amdgpu_buffer_rsrc_t c_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(C, 0, N * M * 4, 0x00020000);   // raw dword buffer over C

    auto load_tile = [&](int tile, v4f (&xv)[UPW][2]) {
#pragma unroll
        for (int s = 0; s < UPW; ++s) {
            int u = wave + s * NW;
            u = u < NUNITS ? u : NUNITS - 1;
            const int bl = (u >> 2) * 2 + ublk;
            int t = tile * TILE_TOK + (u & 3) * 8 + urow;
            t = t < N ? t : N - 1;                     // rows past the end repeat the last row
            const float* src = X + static_cast<int64_t>(t) * K + bl * QK + c4 * 8;
            xv[s][0] = *reinterpret_cast<const v4f_u*>(src);
            xv[s][1] = *reinterpret_cast<const v4f_u*>(src + 4);
        }
    };

    // In-loop form of load_tile.  The vector-memory counter retires in order and counts stores too;
    // the compiler cannot tell how many output stores follow these loads on every path, so it would
    // wait for (nearly) all of them before the quantizer touches the data -- and if the loads were
    // inline assembly with ordinary outputs it would feel free to copy the "results" to other
    // registers before they have arrived.  So the tile in flight lives in the top STAGE registers,
    // which the kernel attribute keeps away from the register allocator: load_tile_async() writes
    // them, take_tile() waits for exactly these loads and only then copies them out.
    constexpr int STAGE = ws_staging_regs(NBLK, NW);
    constexpr int STAGE0 = 256 - STAGE;                // two waves per SIMD: 256 registers each
    static_assert(UPW * 8 <= STAGE, "staging registers hold one tile share");
    // The diagnostic (DUMP) instances leave the fixed registers alone: the extra code of the dumps makes
    // the compiler spill scalar registers into lanes of a vector register of its choosing, which may be
    // one of these.  They read each tile with ordinary loads where the fast instances take it over.
    constexpr bool ASYNC = !DUMP;
    // Instances short of registers rebuild lane-dependent addresses where they are used, from a copy of
    // the lane number the optimizer cannot trace, instead of keeping (or spilling) them across the loop.
    constexpr bool LEAN = STAGE >= 64;
    auto load_tile_async = [&](int tile) {
        if constexpr (!ASYNC) return;
        // the lane's part of the address is rebuilt here once per tile (a few instructions) from a copy of
        // the lane number the optimizer cannot trace, rather than kept in registers across the loop
        int ln = lane;
        asm volatile("" : "+v"(ln));
        const int grp = ln >> 2, c4 = ln & 3;
        const int urow = grp & 7, ublk = grp >> 3;
#pragma unroll
        for (int s = 0; s < UPW; ++s) {
            int u = wave + s * NW;
            u = u < NUNITS ? u : NUNITS - 1;
            const int bl = (u >> 2) * 2 + ublk;
            int t = tile * TILE_TOK + (u & 3) * 8 + urow;
            t = t < N ? t : N - 1;
            const float* src = X + static_cast<int64_t>(t) * K + bl * QK + c4 * 8;
            // the clobber names the top register, which makes the kernel own all 256 of them
            asm volatile("global_load_dwordx4 v[%1:%2], %0, off\n\tglobal_load_dwordx4 v[%3:%4], %0, off offset:16"
                         :: "v"(src), "n"(STAGE0 + 8 * s), "n"(STAGE0 + 8 * s + 3), "n"(STAGE0 + 8 * s + 4), "n"(STAGE0 + 8 * s + 7)
                         : "memory", "v255");
        }
    };
    // `newer` = vector-memory operations issued after load_tile_async: once at most that many are
    // outstanding, its loads have landed.
    auto take_tile = [&](auto newer, int tile, v4f (&xv)[UPW][2]) {
        if constexpr (!ASYNC) {
            load_tile(tile, xv);
            return;
        }
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(decltype(newer)::value) : "memory");
#pragma unroll
        for (int s = 0; s < UPW; ++s) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                float e0, e1, e2, e3;
                asm volatile("v_mov_b32 %0, v[%4]\n\tv_mov_b32 %1, v[%5]\n\tv_mov_b32 %2, v[%6]\n\tv_mov_b32 %3, v[%7]"
                             : "=v"(e0), "=v"(e1), "=v"(e2), "=v"(e3)
                             : "n"(STAGE0 + 8 * s + 4 * h), "n"(STAGE0 + 8 * s + 4 * h + 1), "n"(STAGE0 + 8 * s + 4 * h + 2),
                               "n"(STAGE0 + 8 * s + 4 * h + 3)
                             : "memory");
                xv[s][h] = v4f{e0, e1, e2, e3};
            }
        }
    };

    // The first activation tile is requested before the weights: it has the longer way to come,
    // and it keeps these loads older than at least a tile's worth of later memory operations on
    // every path into the loop, which is what lets the wait in front of the quantizer skip them.
    v4f xv[UPW][2];
    // This work-group's tiles: blockIdx, blockIdx + grid, ... below `ntiles` in full, then -- when the
    // tiles left over by whole rounds are few enough -- one more tile of which it computes a single
    // column tile per wave (tile ntiles + blockIdx / TPW, column part blockIdx % TPW), so that TPW
    // work-groups share each leftover tile instead of a few work-groups running a whole extra round.
    // CSPLIT: the columns are cut into `npart` parts of NW * TPW column tiles and `npart` work-groups share each
    // token tile, one part each.  A work-group then keeps a fraction of the weight (a start-up that is as
    // much shorter) and reads every tile of its group; the members of a group run on one XCD wherever the
    // grid allows (work-groups go to the XCDs in turn), so the tile comes from memory once and from that
    // XCD's L2 for the others.
    int grid = static_cast<int>(gridDim.x);
    int wg = static_cast<int>(blockIdx.x);
    int ct0 = 0;                                       // first column tile of this work-group's part
    if (CSPLIT) {
        const int vid = (grid & 7) == 0 ? (wg & 7) * (grid >> 3) + (wg >> 3) : wg;
        const int group = vid / npart;
        ct0 = (vid - group * npart) * (NW * TPW);
        grid = grid / npart;
        wg = group < grid ? group : ntiles;            // work-groups beyond the last whole group have no tile
    }
    const int n_full = wg < ntiles ? (ntiles - wg + grid - 1) / grid : 0;
    const bool has_part = !CSPLIT && wg < npart;
    const int n_iter = n_full + (has_part ? 1 : 0);
    const int part_col = wg % TPW;
    auto tile_of = [&](int i) { return i < n_full ? wg + i * grid : ntiles + wg / TPW; };
    int tile = tile_of(0);
    if (tid < WS_NBUF) lds_ready[tid] = 0u;
    __syncthreads();                                   // the only barrier of the kernel
    if (n_iter > 0) load_tile(tile, xv);

    // ---- resident weights: fragments of TPW column tiles in registers, their scales in LDS.  All of
    // it is requested here, behind the first activation tile, and consumed after that tile has been
    // quantized: the quantizer runs while the weights are still on their way.
    static_assert(WL >= 0 && WL < TPW, "at least one column tile stays in registers");
    v4i wq[TPW - WL][NBLK];
    v4i* my_wq = lds_wq + static_cast<size_t>(wave) * WL * NBLK * 64 + lane;
    uint2* my_wd = lds_wd + static_cast<size_t>(wave) * TPW * NBLK * 32 + lane;
    auto col_tile_of = [&](int t) {
        const int ct = ct0 + t * NW + wave;            // round t of the waves covers NW adjacent column tiles
        return ct < mct_pad ? ct : mct_pad - 1;        // tiles past the end repeat the last one; never stored
    };
#pragma unroll
    for (int t = 0; t < TPW - WL; ++t) {
#pragma unroll
        for (int b = 0; b < NBLK; ++b)
            wq[t][b] = *reinterpret_cast<const v4i*>(W + (static_cast<size_t>(col_tile_of(t) * NBLK + b) * 64 + lane) * 16);
    }
    // fragments of the column tiles that live in LDS: requested now with the rest, parked in registers that
    // are free until the loop starts, and written to LDS once the first tile has been quantized (requested
    // only then, their whole way from L2 would lie between the quantizer and the first block step)
    v4i wl[WL > 0 ? WL : 1][NBLK];
#pragma unroll
    for (int t = TPW - WL; t < TPW; ++t) {
#pragma unroll
        for (int b = 0; b < NBLK; ++b)
            wl[t - (TPW - WL)][b] = *reinterpret_cast<const v4i*>(W + (static_cast<size_t>(col_tile_of(t) * NBLK + b) * 64 + lane) * 16);
    }
    // scales of one column tile: NBLK x 32 halves, contiguous; a lane takes four at a time
    constexpr int DCHUNKS = NBLK * 8;                  // groups of four halves per column tile
    constexpr int DREP = (DCHUNKS + 63) / 64;
    uint2 draw[TPW][DREP];
    {
        const uint16_t* dplane = reinterpret_cast<const uint16_t*>(W + static_cast<size_t>(mct_pad) * NBLK * 1024);
#pragma unroll
        for (int t = 0; t < TPW; ++t) {
#pragma unroll
            for (int r = 0; r < DREP; ++r) {
                int ci = lane + 64 * r;
                ci = ci < DCHUNKS ? ci : DCHUNKS - 1;
                draw[t][r] = *reinterpret_cast<const uint2*>(dplane + static_cast<size_t>(col_tile_of(t)) * NBLK * 32 + ci * 4);
            }
        }
    }

    // quantizes the tile held in xv into LDS buffer `buf`
    auto quantize_tile = [&](int buf, int tok0, v4f (&xv)[UPW][2]) {
        int ln = lane;
        if (LEAN) asm volatile("" : "+v"(ln));
        const int grp = ln >> 2, c4 = ln & 3;
        const int urow = grp & 7, ublk = grp >> 3;
#pragma unroll
        for (int s = 0; s < UPW; ++s) {
            const int u = wave + s * NW;
            if (u >= NUNITS) break;                    // wave-uniform
            const int row = (u & 3) * 8 + urow;
            const int bl = (u >> 2) * 2 + ublk;
            const v4f x0 = xv[s][0], x1 = xv[s][1];
            const BlockQuant bq = (relu & 1) ? quantize_block_lane<Q81, true>(x0, x1) : quantize_block_lane<Q81, false>(x0, x1);
            uint2* dst = reinterpret_cast<uint2*>(lds_a[buf]) + ((bl * 64 + (c4 >> 1) * 32 + row) * 2 + (c4 & 1));
            *dst = uint2{bq.q_lo, bq.q_hi};
            if (c4 == 0) lds_d[buf][bl * 32 + row] = uint2{bq.d_bits, 0u};
            if (DUMP && xq_dump) {
                const int t = tok0 + row;
                if (t < N) store_block_part(xq_dump + (static_cast<int64_t>(t) * NBLK + bl) * Q8_0_BYTES, c4, bq);
            }
        }
    };

    // A wave announces that its share of a quantized tile is in LDS; consumers poll the count.  The
    // LDS unit executes one wave's operations in order, so the count becomes visible after the data.
    auto announce = [&](int buf) {
        asm volatile("" ::: "memory");
        if (lane == 0) __hip_atomic_fetch_add(&lds_ready[buf], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        asm volatile("" ::: "memory");
    };
    auto await_tile = [&](int buf, unsigned want) {
        while (__hip_atomic_load(&lds_ready[buf], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < want)
            __builtin_amdgcn_s_sleep(1);
        asm volatile("" ::: "memory");
    };

    if (n_iter > 0) {
        quantize_tile(0, tile * TILE_TOK, xv);
        announce(0);
    }
    // weight scales and the fragments that live in LDS: written and read by this wave only
#pragma unroll
    for (int t = 0; t < TPW; ++t) {
#pragma unroll
        for (int r = 0; r < DREP; ++r) {
            const int ci = lane + 64 * r;
            if (ci < DCHUNKS) {
                const uint2 h4 = draw[t][r];
                v4i* dst = reinterpret_cast<v4i*>(my_wd - lane + t * NBLK * 32 + ci * 4);
                dst[0] = v4i{static_cast<int>(h4.x & 0xffffu), 0, static_cast<int>(h4.x >> 16), 0};
                dst[1] = v4i{static_cast<int>(h4.y & 0xffffu), 0, static_cast<int>(h4.y >> 16), 0};
            }
        }
    }
#pragma unroll
    for (int t = TPW - WL; t < TPW; ++t) {
#pragma unroll
        for (int b = 0; b < NBLK; ++b)
            my_wq[((t - (TPW - WL)) * NBLK + b) * 64] = wl[t - (TPW - WL)][b];
    }
    // Every weight fragment has arrived before the loop starts: a load still pending here would make
    // its first use inside the loop wait for vmcnt(0), i.e. for all output stores, on every iteration.
    __builtin_amdgcn_s_waitcnt(0x0f70);                // vmcnt(0), other counters untouched
    // the second tile is requested now and quantized during the first one (at QSTEP_TILE, below)
    if (n_iter > 1) load_tile_async(tile_of(1));

    // Step at which the next tile is quantized.  Its loads were issued one full round of column tiles
    // earlier (right after the previous quantization freed the staging registers), so they have
    // long arrived; the tile after it is requested as soon as this one is in LDS.
    // QEARLY: at the very start of the tile instead.  The sooner the next tile is announced, the less the waves wait for
    // each other where one tile ends and the next begins; but in the first iteration the next tile's loads have only
    // just been issued, and waiting for them there costs a work-group with one or two tiles more than it gains later
    // (us, two thirds in / at the start: 26368 x 256 -> 768  22.7 / 21.8, 52736 rows 40.6 / 40.1, 13184 rows 12.8 / 13.1;
    // 26368 x 128 -> 768  17.7 / 18.3): the launcher picks it for K = 256 with three column tiles per wave from three
    // whole rounds of tiles on.
    constexpr int QSTEP_TILE = QEARLY ? 0 : (2 * TPW) / 3;   // column tile in front of which the next tile is quantized
    constexpr int QSTEP = QSTEP_TILE * NBLK;
    // Vector-memory operations issued between a tile's loads and the wait in front of its
    // quantization: 16 stores per column tile, one round of column tiles (fewer before the first wait).
    constexpr int NEWER_FIRST = 16 * (QSTEP / NBLK) < 63 ? 16 * (QSTEP / NBLK) : 63;
    constexpr int NEWER = 16 * TPW < 63 ? 16 * TPW : 63;

    // Block sums leave the matrix pipe as floats.  An int8 MFMA that starts from the bit pattern of
    // 1.5 * 2^23 instead of zero returns, read as binary32, exactly 1.5 * 2^23 + sum (|sum| <= 32 * 128 * 128
    // stays inside that binade, where one unit in the last place is one); a bf16 MFMA whose only non-zero
    // products are (-0.75 * 2^23) * 1 in k slots 0 and 4 then takes the offset off again, exactly, since
    // float(sum) is representable.  This replaces one v_cvt_f32_i32 per output and block on the vector
    // pipe, which is what bounds this kernel, by 8 passes of the matrix pipe, which has the slack.
    // The constants are hidden from the optimizer so that they stay in registers instead of being
    // rebuilt in front of every MFMA.
    v16i magic_i;
#pragma unroll
    for (int r = 0; r < 16; ++r) magic_i[r] = WS_MAGIC_BITS;
    asm volatile("" : "+v"(magic_i));
    typedef short v4s __attribute__((ext_vector_type(4)));
    v4s unbias_a = {static_cast<short>(0xCAC0), 0, 0, 0};   // bf16 -0.75 * 2^23
    v4s unbias_b = {static_cast<short>(0x3F80), 0, 0, 0};   // bf16 1
    asm volatile("" : "+v"(unbias_a), "+v"(unbias_b));

    // No barrier inside the loop.  A wave may start tile `it` once all waves have announced it, which
    // also means all of them have reached the quantization point of tile it-1, i.e. have left tile it-2; the tile quantized during tile `it`
    // goes to buffer (it+1) % 3, last read for tile it-2, which every wave has left by then.
    for (int it = 0; it < n_iter; ++it) {
        tile = tile_of(it);
        const int buf = it % WS_NBUF;
        const int tok0 = tile * TILE_TOK;
        const bool has_next = it + 1 < n_iter;
        const int next = has_next ? tile_of(it + 1) : tile;
        const bool partial = it >= n_full;             // compute column tile part_col only
        await_tile(buf, static_cast<unsigned>(NW) * static_cast<unsigned>(it / WS_NBUF + 1));

        // ---------------- MFMA one block ahead of the settle; tiles in turn, blocks ascending
        // Per pair of blocks: two int8 MFMAs (exact block sums, one result buffer per parity) and one
        // v_mfma_f32_32x32x4_2b_f16 whose two 32x32 outer products are the scale tables
        // d_a[row] * d_w[col] of both blocks: the scale sits in the first of a lane's four k slots and
        // the others hold zero, so each entry is the exact binary32 product of two halves.  (The
        // half-precision form shares the matrix pipe with the int8 MFMAs and runs beside vector
        // instructions; the single-precision form would hold up the vector pipe.)
        v16i sum_a, sum_b;
        v32f scl;
        v32f zero_f2;
#pragma unroll
        for (int r = 0; r < 32; ++r) zero_f2[r] = 0.0f;
        v16f acc;
        // LDS operands of one pair of steps, fetched a pair ahead of the MFMAs that consume them
        struct PairOps { v4i a0, a1, w0, w1; uint2 da, dw; };
        auto fetch_pair = [&](int st, PairOps& o) {
            const int t = st / NBLK, b = st % NBLK;
            o.a0 = lds_a[buf][b * 64 + lane];
            o.a1 = lds_a[buf][(b + 1) * 64 + lane];
            o.da = lds_d[buf][b * 32 + lane];          // lanes 0..31: rows of block b, 32..63: of block b + 1
            o.dw = my_wd[(t * NBLK + b) * 32];
            if (t >= TPW - WL) {
                o.w0 = my_wq[((t - (TPW - WL)) * NBLK + b) * 64];
                o.w1 = my_wq[((t - (TPW - WL)) * NBLK + b + 1) * 64];
            }
        };
        // CT0 (C stored [M][N], features outermost): the operands change places, in the block sums and in the scale
        // tables alike, so that a lane holds one token and sixteen features instead of one feature and sixteen tokens
        // and a half-wave store is again one line of a C row.  Both operands of these MFMAs have the same fragment
        // layout (lane % 32 = row or column, lane / 32 = half of k), the products and their order of addition are the
        // same: same bits.
        auto scale_tables = [&](const uint2& da, const uint2& dw) {
            typedef _Float16 v4h __attribute__((ext_vector_type(4)));
            if constexpr (CT0) return __builtin_amdgcn_mfma_f32_32x32x4f16(__builtin_bit_cast(v4h, dw), __builtin_bit_cast(v4h, da), zero_f2, 0, 0, 0);
            else return __builtin_amdgcn_mfma_f32_32x32x4f16(__builtin_bit_cast(v4h, da), __builtin_bit_cast(v4h, dw), zero_f2, 0, 0, 0);
        };
        auto block_sum = [&](int st, const v4i& a, const v4i& w_lds) {
            const int t = st / NBLK, b = st % NBLK;
            const v4i w = t < TPW - WL ? wq[t < TPW - WL ? t : 0][b] : w_lds;
            if constexpr (CT0) return __builtin_amdgcn_mfma_i32_32x32x32_i8(w, a, magic_i, 0, 0, 0);
            else return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, w, magic_i, 0, 0, 0);
        };
        // 1.5 * 2^23 + sum -> float(sum), on the matrix pipe
        auto to_float = [&](const v16i& biased) {
            return __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(unbias_a, unbias_b, __builtin_bit_cast(v16f, biased), 0, 0, 0);
        };
        auto settle = [&](int st, const v16f& sum, const v16f scl) {
            const int t = st / NBLK, b = st % NBLK;
            if (b == 0) {
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[r] = __builtin_fmaf(sum[r], scl[r], 0.0f);
            } else {
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[r] = __builtin_fmaf(sum[r], scl[r], acc[r]);
            }
            const int m = (ct0 + t * NW + wave) * 32 + (CT0 ? 0 : j);   // this lane's output feature (CT0: the first of its column tile)
            if (DUMP && sums_dump) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int tok = CT0 ? tok0 + j : tok0 + mfma32_row(r, lane);
                    const int mm = CT0 ? m + mfma32_row(r, lane) : m;
                    if (tok < N && mm < M) sums_dump[(static_cast<int64_t>(tok) * M + mm) * NBLK + b] = static_cast<int>(sum[r]);
                }
            }
            if (b == NBLK - 1) {
                // The tile is complete: each half-wave store writes one full 128-byte line of a C
                // row.  Buffer stores with a bounds-checked offset: lanes past the edge of C pass an
                // offset beyond the buffer and are dropped by the hardware, so every wave issues
                // exactly 16 stores here and the memory counter stays predictable.
                // The whole byte offset of a store sits in the vector operand, which is what the hardware checks
                // against the size of C: rows past the last token lie behind the end of the buffer and drop out
                // by themselves (the ragged last tile needs no predicates), columns past M start from an offset of
                // 2^31, which stays outside whatever is added to it (C is below 2^31 bytes, see the launcher).
                // Stepping the offset costs one add per store; a scalar offset per row would cost none but is not
                // range-checked, and its sixteen predicates per column tile ran for every tile, ragged or not.
                // CT0: rows of C are features.  The lane's token picks the column, tokens past the end start from 2^31;
                // feature rows past M lie behind the end of the buffer (the launcher keeps the padded height of C
                // below 2^31 bytes, so the offsets of live lanes do not wrap), and column tiles past the padded end,
                // which repeat the last tile's weights, start from 2^31 like the tokens.
                uint32_t off;
                if constexpr (CT0)
                    off = (tok0 + j < N && m < mct_pad * 32) ? (static_cast<uint32_t>(m + 4 * hh) * N + (tok0 + j)) * 4u : 0x80000000u;
                else
                    off = m < M ? (static_cast<uint32_t>(tok0 + 4 * hh) * M + m) * 4u : 0x80000000u;
                int pitch = (CT0 ? N : M) * 4;
                asm volatile("" : "+s"(pitch));          // one scalar, not sixteen folded row offsets
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(acc[r]), c_rsrc, off, 0, WS_STORE_AUX);
                    off += ((r & 3) == 3 ? 5 : 1) * pitch;   // rows 8 * (r / 4) + r % 4 (+ 4 in the upper half-wave)
                }
            }
        };
        static_assert(STEPS % 2 == 0, "steps are taken in pairs");
#pragma unroll
        for (int t0 = 0; t0 < TPW; ++t0) {
            // One basic block per column tile (see opaque_one()): the accumulator is born and stored
            // inside it, so nothing but loop state crosses the boundary.
            if (!opaque_one()) continue;
            if (partial && t0 != part_col) continue;
            // QEARLY: half of the waves quantize at the start of the tile, the other half one column tile later, so
            // that not all eight are at their vector work at once (another 1 to 2 % at 26368 x 256 -> 768; which waves
            // form a half makes no difference, two column tiles later gains nothing).  Sixteen stores lie between the
            // loads and the first wait of the second half.
            const bool q_here = QEARLY ? ((t0 == 0 && wave < NW / 2) || (t0 == 1 && wave >= NW / 2)) : t0 == QSTEP_TILE;
            if (q_here && has_next) {
                {
                    v4f xn[UPW][2];
                    if (it == 0) {
                        if (QEARLY && t0 == 1) take_tile(std::integral_constant<int, 16>{}, next, xn);
                        else take_tile(std::integral_constant<int, NEWER_FIRST>{}, next, xn);
                    }
                    else take_tile(std::integral_constant<int, NEWER>{}, next, xn);
                    if (it + 2 < n_iter) load_tile_async(tile_of(it + 2));
                    quantize_tile((it + 1) % WS_NBUF, next * TILE_TOK, xn);
                    announce((it + 1) % WS_NBUF);
                }
            }
            // Pairs of steps use the operand sets pe / po alternately, so they swap roles by name.  A
            // pair starts by issuing its scale MFMA and the block sum of its second step; the block
            // sum of the next pair's first step follows the first settle.  The barriers keep the
            // compiler from sinking MFMAs next to their consumers, where every settle would wait
            // out a whole MFMA; the one wait left per pair (for the scale table) is covered by the
            // other wave of the SIMD.
            PairOps pe, po;
            const int s0 = t0 * NBLK;
            // Beside 64 staging registers there is no room for a second operand set: one set, refilled as
            // soon as its MFMAs are issued.
            constexpr bool TWO_SETS = !LEAN;
            fetch_pair(s0, pe);
            if (TWO_SETS && NBLK > 2) fetch_pair(s0 + 2, po);
            if (TWO_SETS) sum_a = block_sum(s0, pe.a0, pe.w0);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int pr = 0; pr < NBLK / 2; ++pr) {
                const int st = s0 + 2 * pr;
                if constexpr (TWO_SETS) {
                    PairOps& cur = (pr & 1) ? po : pe;
                    PairOps& nxt = (pr & 1) ? pe : po;
                    const v16f flt_a = to_float(sum_a);
                    scl = scale_tables(cur.da, cur.dw);
                    sum_b = block_sum(st + 1, cur.a1, cur.w1);
                    __builtin_amdgcn_sched_barrier(0);
                    settle(st, flt_a, __builtin_shufflevector(scl, scl, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15));
                    __builtin_amdgcn_sched_barrier(0);
                    const v16f flt_b = to_float(sum_b);
                    if (2 * pr + 2 < NBLK) sum_a = block_sum(st + 2, nxt.a0, nxt.w0);
                    if (2 * pr + 4 < NBLK) fetch_pair(st + 4, cur);
                    __builtin_amdgcn_sched_barrier(0);
                    settle(st + 1, flt_b, __builtin_shufflevector(scl, scl, 16, 17, 18, 19, 20, 21, 22, 23, 24, 25, 26, 27, 28, 29, 30, 31));
                    __builtin_amdgcn_sched_barrier(0);
                } else {
                    // one block sum alive at a time; the other wave of the SIMD fills the waits
                    sum_a = block_sum(st, pe.a0, pe.w0);
                    scl = scale_tables(pe.da, pe.dw);
                    const v16f flt_a = to_float(sum_a);
                    __builtin_amdgcn_sched_barrier(0);
                    settle(st, flt_a, __builtin_shufflevector(scl, scl, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15));
                    __builtin_amdgcn_sched_barrier(0);
                    sum_a = block_sum(st + 1, pe.a1, pe.w1);
                    if (2 * pr + 2 < NBLK) fetch_pair(st + 2, pe);
                    const v16f flt_b = to_float(sum_a);
                    __builtin_amdgcn_sched_barrier(0);
                    settle(st + 1, flt_b, __builtin_shufflevector(scl, scl, 16, 17, 18, 19, 20, 21, 22, 23, 24, 25, 26, 27, 28, 29, 30, 31));
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    }
}

// The attribute takes a literal, hence one kernel per staging size (16 registers up to K = 256, 32 or
// 64 beyond).  On this target the register allocator's budget is TWICE the attribute's value (the
// value counts architectural and accumulation registers separately): 120 keeps it below v240.  A
// value the compiler does not honour would go unnoticed until its registers and the staged tile
// collide, so the build checks the generated code (check_ws_isa.py).
template <int NW, int TPW, int NBLK, int WL, bool DUMP, bool Q81, bool CSPLIT, bool QEARLY = false, bool CT0 = false>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(2, 2), amdgpu_num_vgpr(120)))
void q8_linear_ws_kernel(const uint8_t* __restrict__ W, const float* __restrict__ X, float* __restrict__ C,
                         int M, int N, int ntiles, int npart, int relu, uint8_t* __restrict__ xq_dump,
                         int32_t* __restrict__ sums_dump) {
    static_assert(ws_compiler_vgprs(NBLK, NW) == 2 * 120, "staging size");
    q8_linear_ws_body<NW, TPW, NBLK, WL, DUMP, Q81, CSPLIT, QEARLY, CT0>(W, X, C, M, N, ntiles, npart, relu, xq_dump, sums_dump);
}
template <int NW, int TPW, int NBLK, int WL, bool DUMP, bool Q81, bool CSPLIT, bool QEARLY = false, bool CT0 = false>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(2, 2), amdgpu_num_vgpr(112)))
void q8_linear_ws32_kernel(const uint8_t* __restrict__ W, const float* __restrict__ X, float* __restrict__ C,
                           int M, int N, int ntiles, int npart, int relu, uint8_t* __restrict__ xq_dump,
                           int32_t* __restrict__ sums_dump) {
    static_assert(ws_compiler_vgprs(NBLK, NW) == 2 * 112, "staging size");
    q8_linear_ws_body<NW, TPW, NBLK, WL, DUMP, Q81, CSPLIT, QEARLY, CT0>(W, X, C, M, N, ntiles, npart, relu, xq_dump, sums_dump);
}

template <int NW, int TPW, int NBLK, int WL, bool DUMP, bool Q81, bool CSPLIT, bool QEARLY = false, bool CT0 = false>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(2, 2), amdgpu_num_vgpr(96)))
void q8_linear_ws64_kernel(const uint8_t* __restrict__ W, const float* __restrict__ X, float* __restrict__ C,
                           int M, int N, int ntiles, int npart, int relu, uint8_t* __restrict__ xq_dump,
                           int32_t* __restrict__ sums_dump) {
    static_assert(ws_compiler_vgprs(NBLK, NW) == 2 * 96, "staging size");
    q8_linear_ws_body<NW, TPW, NBLK, WL, DUMP, Q81, CSPLIT, QEARLY, CT0>(W, X, C, M, N, ntiles, npart, relu, xq_dump, sums_dump);
}

template <int TPW, int NBLK, int WL, int NW, bool Q81, bool CSPLIT = false, bool CT0 = false>
int launch_q8_linear_ws(const void* W, const float* X, float* C, int M, int N, int relu,
                        void* xq_dump, int32_t* sums_dump, hipStream_t stream, int cparts = 1) {
    // Eight waves fill a CU (256 registers each): one resident work-group of 8 waves per CU, or two
    // of 4.  With more tiles than resident work-groups every work-group takes the same number of
    // tiles (824 tiles on 256 CUs: 206 work-groups x 4 rather than 256 x 3 + 56 x 1).
    const int cus = device_cu_count() * (NW == 4 ? 2 : 1);
    const int all_tiles = (N + TILE_TOK - 1) / TILE_TOK;
    int wgs, ntiles = all_tiles, npart = 0;
    const int left = all_tiles % cus;
    if (CSPLIT) {
        // one work-group per CU; `cparts` of them share a token tile, a column part each
        wgs = cus;
        npart = cparts;
    } else if (all_tiles > cus && left > 0 && left * TPW <= cus && TPW > 1) {
        // whole rounds on every CU, then the leftover tiles shared by TPW work-groups each
        wgs = cus;
        ntiles = all_tiles - left;
        npart = left * TPW;
    } else {
        const int rounds = (all_tiles + cus - 1) / cus;
        wgs = (all_tiles + rounds - 1) / rounds;
    }
    const dim3 grid(wgs), block(NW * 64);
    constexpr size_t lds = static_cast<size_t>(WS_NBUF) * NBLK * (1024 + 256) + static_cast<size_t>(NW) * TPW * NBLK * 256 + 16 +
                           static_cast<size_t>(NW) * WL * NBLK * 1024;
    using KernelFn = void (*)(const uint8_t*, const float*, float*, int, int, int, int, int, uint8_t*, int32_t*);
    KernelFn fast, dump;
    // the next tile quantized at the start of a tile rather than two thirds in (see QEARLY in the kernel)
    constexpr bool CAN_EARLY = TPW == 3 && NBLK == 8 && NW == 8 && !CSPLIT;
    const bool early = CAN_EARLY && all_tiles / cus >= 3;
    if constexpr (CT0) {
        // C with the features outermost: the fast instances only (a call that asks for the diagnostic buffers
        // takes the general kernel, see try_q8_linear_ws)
        static_assert(!CSPLIT, "no column parts for this orientation");
        if constexpr (CAN_EARLY) {
            fast = early ? &q8_linear_ws_kernel<NW, TPW, NBLK, WL, false, Q81, false, true, true> : &q8_linear_ws_kernel<NW, TPW, NBLK, WL, false, Q81, false, false, true>;
        } else if constexpr (ws_staging_regs(NBLK, NW) == 16) {
            fast = &q8_linear_ws_kernel<NW, TPW, NBLK, WL, false, Q81, false, false, true>;
        } else if constexpr (ws_staging_regs(NBLK, NW) == 32) {
            fast = &q8_linear_ws32_kernel<NW, TPW, NBLK, WL, false, Q81, false, false, true>;
        } else {
            static_assert(ws_staging_regs(NBLK, NW) == 64, "no kernel for this staging size");
            fast = &q8_linear_ws64_kernel<NW, TPW, NBLK, WL, false, Q81, false, false, true>;
        }
        dump = fast;
    } else if constexpr (CAN_EARLY) {
        static_assert(ws_staging_regs(NBLK, NW) == 16, "the instance with the early quantization");
        fast = early ? &q8_linear_ws_kernel<NW, TPW, NBLK, WL, false, Q81, CSPLIT, true> : &q8_linear_ws_kernel<NW, TPW, NBLK, WL, false, Q81, CSPLIT>;
        dump = early ? &q8_linear_ws_kernel<NW, TPW, NBLK, WL, true, Q81, CSPLIT, true> : &q8_linear_ws_kernel<NW, TPW, NBLK, WL, true, Q81, CSPLIT>;
    } else if constexpr (ws_staging_regs(NBLK, NW) == 16) {
        fast = &q8_linear_ws_kernel<NW, TPW, NBLK, WL, false, Q81, CSPLIT>;
        dump = &q8_linear_ws_kernel<NW, TPW, NBLK, WL, true, Q81, CSPLIT>;
    } else if constexpr (ws_staging_regs(NBLK, NW) == 32) {
        fast = &q8_linear_ws32_kernel<NW, TPW, NBLK, WL, false, Q81, CSPLIT>;
        dump = &q8_linear_ws32_kernel<NW, TPW, NBLK, WL, true, Q81, CSPLIT>;
    } else {
        static_assert(ws_staging_regs(NBLK, NW) == 64, "no kernel for this staging size");
        fast = &q8_linear_ws64_kernel<NW, TPW, NBLK, WL, false, Q81, CSPLIT>;
        dump = &q8_linear_ws64_kernel<NW, TPW, NBLK, WL, true, Q81, CSPLIT>;
    }
    if (lds > 64 * 1024) {
        // (once per instance; where the launcher chooses between two forms of the kernel, once per form)
        static hipError_t attr_fast[2] = {hipErrorNotReady, hipErrorNotReady}, attr_dump[2] = {hipErrorNotReady, hipErrorNotReady};
        static std::mutex attr_lock;
        {
            std::lock_guard<std::mutex> hold(attr_lock);
            if (attr_fast[early] == hipErrorNotReady) {
                attr_fast[early] = hipFuncSetAttribute(reinterpret_cast<const void*>(fast), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
                attr_dump[early] = hipFuncSetAttribute(reinterpret_cast<const void*>(dump), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
            }
        }
        if (attr_fast[early] != hipSuccess || attr_dump[early] != hipSuccess) {
            (void)hipGetLastError();
            return -1;                                  // fall back to the general kernel
        }
    }
    if (xq_dump || sums_dump)
        hipLaunchKernelGGL(dump, grid, block, lds, stream, static_cast<const uint8_t*>(W), X, C, M, N, ntiles, npart, relu,
                           static_cast<uint8_t*>(xq_dump), sums_dump);
    else
        hipLaunchKernelGGL(fast, grid, block, lds, stream, static_cast<const uint8_t*>(W), X, C, M, N, ntiles, npart, relu,
                           static_cast<uint8_t*>(nullptr), static_cast<int32_t*>(nullptr));
    return check_launch("q8_linear_ws_kernel");
}

// returns -1 when the shape has no weight-stationary instance
// `csplit`: -1 never, 1 wherever there is an instance, 0 by the gate below
template <bool Q81, bool CT0 = false>
int try_q8_linear_ws(const void* W, const float* X, float* C, int M, int N, int nblk, int c_trans,
                     int relu, int csplit, void* xq_dump, int32_t* sums_dump, hipStream_t stream) {
    if (!c_trans && !CT0) {
        // C [M][N] (the weight was src[0]): instances of their own, without the diagnostic buffers
        if (xq_dump || sums_dump) return -1;
        return try_q8_linear_ws<Q81, true>(W, X, C, M, N, nblk, 0, relu, -1, nullptr, nullptr, stream);
    }
    // the kernel addresses C with 32-bit byte offsets; with the features outermost the offsets it forms reach
    // the padded height of C plus the four rows between the two halves of a wave
    if (static_cast<int64_t>(N) * M * 4 >= 0x7fff0000LL) return -1;
    if (CT0 && static_cast<int64_t>(N) * (packed_tiles(M) * 32 + 4) * 4 >= 0x7fff0000LL) return -1;
    const int mct = (M + 31) / 32;
    const int tpw = (mct + 7) / 8;
    if (CT0) csplit = -1;
    // Column parts: `tpw` work-groups of the one-column-tile-per-wave instance share each token tile.  Every
    // work-group then quantizes the whole tile for a `tpw`-th of the columns, which costs more than the shorter
    // start-up saves except where the whole-width instance is short of registers and LDS (measured, us, parts /
    // whole: 26368 x 256 -> 768  23.8 / 22.2;  10609 x 128 -> 512  6.8 / 6.3;  26368 x 128 -> 1024  20.1 / 25.1).
    if (!CT0 && tpw > 1 && csplit >= 0) {
        const int cus = device_cu_count();
        const int tiles = (N + TILE_TOK - 1) / TILE_TOK;
        // ... and wherever there is no whole-width instance at all (K = 128 beyond 1024 columns, K = 256 beyond 768): the
        // parts take any width (a work-group holds 256 columns, `tpw` of them share a tile), the alternative is the
        // general kernel, which streams the weight per tile (10609 x 256 -> 1024: 15.4 us in parts, 31.6 general)
        const bool no_whole = (nblk == 4 && tpw > 4) || (nblk == 8 && tpw > 3);
        const bool take = csplit > 0 || (tpw == 4 && tiles >= 3 * cus) || no_whole;
        if (take && cus >= tpw) {
#define PPML_WSC(NBLK) return launch_q8_linear_ws<1, NBLK, 0, 8, Q81, true>(W, X, C, M, N, relu, xq_dump, sums_dump, stream, tpw)
            if (nblk == 4) PPML_WSC(4);
            if (nblk == 8) PPML_WSC(8);
#undef PPML_WSC
        }
    }
#define PPML_WS(TPW, NBLK, WL, NW) return launch_q8_linear_ws<TPW, NBLK, WL, NW, Q81, false, CT0>(W, X, C, M, N, relu, xq_dump, sums_dump, stream)
    // Up to four column tiles: work-groups of four waves, one column tile each and two per CU, so no
    // wave idles (with eight waves half of them would have no column tile).
    if (mct <= 4) {
        if (nblk == 2) PPML_WS(1, 2, 0, 4);
        if (nblk == 4) PPML_WS(1, 4, 0, 4);
        if (nblk == 8) PPML_WS(1, 8, 0, 4);
        if (nblk == 16) PPML_WS(1, 16, 0, 4);
    }
    // (column tiles per wave, blocks of K, column tiles whose fragments live in LDS instead of registers)
    if (nblk == 2) {                                   // K = 64: the 64 -> 64 and 64 -> 256 projections of the full-MSA track
        if (tpw == 1) PPML_WS(1, 2, 0, 8);
    } else if (nblk == 4) {
        if (tpw == 1) PPML_WS(1, 4, 0, 8);
        if (tpw == 2) PPML_WS(2, 4, 0, 8);
        if (tpw == 3) PPML_WS(3, 4, 0, 8);
        if (tpw == 4) PPML_WS(4, 4, 0, 8);
    } else if (nblk == 8) {
        if (tpw == 1) PPML_WS(1, 8, 0, 8);
        if (tpw == 2) PPML_WS(2, 8, 0, 8);
        if (tpw == 3) PPML_WS(3, 8, 1, 8);
    } else if (nblk == 16) {
        if (tpw == 1) PPML_WS(1, 16, 0, 8);
    }
#undef PPML_WS
    return -1;
}

// ------------------------------------------------------------------------------------------
// Low-latency form of the same linear, for Q8_0M weights of at most 64 Ki elements and so few tokens that
// a work-group of the weight-stationary kernel gets one or two token tiles: there is nothing to amortise
// resident weights over, and one tile per work-group is a chain of load -> quantize -> block steps ->
// store in which nothing overlaps (measured at 10609 x 512 -> 128: 12.4 us against about 8 us for a copy
// of the same bytes).  Here the tokens are cut into units of TOK = 8 or 16 rows (32 at two per CU), one four-wave work-group
// each, three of them resident per CU at different stages:
//
//   * every lane requests its whole share of the unit's activations at once (with all work-groups
//     resident the whole of X is in flight within the first microsecond), and right behind them ALL the
//     weight fragments and scales of its wave's CPW column tiles (wave, wave + 4, ...): at most 64 + 8
//     registers, served by L2 (the weight is a few tens of KB shared by every work-group) while the
//     activations are still on their way from HBM;
//   * the unit is quantized into LDS in MFMA-fragment order as its loads land; one barrier;
//   * per column tile and pair of blocks: two v_mfma_i32_32x32x32_i8 and one v_mfma_f32_32x32x4_2b_f16 for
//     the two scale tables, no memory operation but the LDS reads.  The activations are the A operand, so
//     the TOK tokens occupy the first TOK / 2 accumulator registers of every lane and only those are
//     settled and stored: the matrix pipe does 32 / TOK times the useful work (it has the slack: these
//     shapes are bound by memory and latency), the vector pipe none extra.
//
// Blocks ascend per output and every settlement is the same fma as everywhere else: same bits.
// ------------------------------------------------------------------------------------------
template <int TOK, int NBLK, int CPW, bool DUMP, bool Q81>
__device__ __forceinline__ void q8_linear_ll_body(
    const uint8_t* __restrict__ W, const float* __restrict__ X, float* __restrict__ C,
    int M, int N, int relu, uint8_t* __restrict__ xq_dump, int32_t* __restrict__ sums_dump) {
    static_assert(TOK == 8 || TOK == 16 || TOK == 32, "token rows per work-group");
    static_assert(NBLK % 2 == 0, "blocks are taken in pairs");
    static_assert(CPW * NBLK <= 16, "the wave's weight fragments stay in 64 registers");
    constexpr int NW = 4;
    constexpr int K = NBLK * QK;
    constexpr int NUNITS = (TOK / 8) * (NBLK / 2);     // (8 rows) x (2 blocks) each: one wave-wide load pair
    constexpr int UPW = (NUNITS + NW - 1) / NW;
    constexpr int RV = TOK / 2;                        // accumulator registers that hold real tokens
    __shared__ __attribute__((aligned(16))) v4i lds_a[NBLK * 64];     // [block][k half][row][16 quants]
    __shared__ __attribute__((aligned(8))) uint2 lds_d[NBLK * 32];    // [block][row] {fp16 scale, 0, 0, 0}
    __shared__ uint16_t lds_wd[NW * CPW * (NBLK / 2) * 64];           // [wave][column tile][pair][lane] fp16 weight scales

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 31;
    const int tok0 = blockIdx.x * TOK;
    const int mct = (M + 31) / 32;
    const int mct_pad = packed_tiles(M);
    const int grp = lane >> 2, c4 = lane & 3;
    const int urow = grp & 7, ublk = grp >> 3;

    // ---- all of this lane's activations at once
    v4f xv[UPW][2];
#pragma unroll
    for (int s = 0; s < UPW; ++s) {
        int u = wave + s * NW;
        u = u < NUNITS ? u : NUNITS - 1;               // surplus slots repeat the last unit
        const int bl = (u / (TOK / 8)) * 2 + ublk;
        int t = tok0 + (u % (TOK / 8)) * 8 + urow;
        t = t < N ? t : N - 1;                         // rows past the end repeat the last row; never stored
        const float* src = X + static_cast<int64_t>(t) * K + bl * QK + c4 * 8;
        xv[s][0] = *reinterpret_cast<const v4f_u*>(src);
        xv[s][1] = *reinterpret_cast<const v4f_u*>(src + 4);
    }
    // ---- all weight fragments and scales of this wave's column tiles, behind them
    v4i wq[CPW][NBLK];
    uint16_t wd[CPW][NBLK / 2];                        // parked in LDS once they have arrived: read back pair by pair
    {
        const uint16_t* dplane = reinterpret_cast<const uint16_t*>(W + static_cast<size_t>(mct_pad) * NBLK * 1024);
#pragma unroll
        for (int t = 0; t < CPW; ++t) {
            int ct = wave + t * NW;
            ct = ct < mct_pad ? ct : mct_pad - 1;      // tiles past the end repeat the last one; never stored
            const size_t frag = static_cast<size_t>(ct) * NBLK;
#pragma unroll
            for (int b = 0; b < NBLK; ++b) wq[t][b] = *reinterpret_cast<const v4i*>(W + ((frag + b) * 64 + lane) * 16);
#pragma unroll
            for (int pr = 0; pr < NBLK / 2; ++pr)      // lanes 0..31: columns of block 2 pr, 32..63: of block 2 pr + 1
                wd[t][pr] = dplane[(frag + 2 * pr) * 32 + lane];
        }
    }

    // ---- quantize into LDS
#pragma unroll
    for (int s = 0; s < UPW; ++s) {
        const int u = wave + s * NW;
        if (u >= NUNITS) break;                        // wave-uniform
        const int row = (u % (TOK / 8)) * 8 + urow;
        const int bl = (u / (TOK / 8)) * 2 + ublk;
        const v4f x0 = xv[s][0], x1 = xv[s][1];
        const BlockQuant bq = relu ? quantize_block_lane<Q81, true>(x0, x1) : quantize_block_lane<Q81, false>(x0, x1);
        uint2* dst = reinterpret_cast<uint2*>(lds_a) + ((bl * 64 + (c4 >> 1) * 32 + row) * 2 + (c4 & 1));
        *dst = uint2{bq.q_lo, bq.q_hi};
        if (c4 == 0) lds_d[bl * 32 + row] = uint2{bq.d_bits, 0u};
        if (DUMP && xq_dump) {
            const int t = tok0 + row;
            if (t < N) store_block_part(xq_dump + (static_cast<int64_t>(t) * NBLK + bl) * Q8_0_BYTES, c4, bq);
        }
    }
    uint16_t* my_wd = lds_wd + wave * (CPW * (NBLK / 2) * 64) + lane;
#pragma unroll
    for (int t = 0; t < CPW; ++t)
#pragma unroll
        for (int pr = 0; pr < NBLK / 2; ++pr) my_wd[(t * (NBLK / 2) + pr) * 64] = wd[t][pr];   // written and read by this wave only
    __syncthreads();

    // ---- column tiles of this wave, blocks ascending.  (The block sums are converted on the vector pipe here: the
    // matrix-pipe conversion of the weight-stationary kernel costs twenty registers, which this kernel, at three
    // waves per SIMD, spends on the operands fetched ahead instead; measured equal at 10609 x 512 -> 128 and
    // better on the few-token shapes.)
    v32f zero_f;
#pragma unroll
    for (int r = 0; r < 32; ++r) zero_f[r] = 0.0f;
    typedef _Float16 v4h __attribute__((ext_vector_type(4)));
    // LDS operands of one pair of blocks.  They are fetched a pair ahead, under the matrix work of the pair in hand:
    // with the work-groups of a CU at different stages the LDS round trip used to be covered by other waves, but the
    // work-groups whose activations arrive last run alone, and their chain of pairs is what the kernel ends on
    // (per-wave time stamps: 2.1 us for the sixteen blocks of the pair feed-forward down-projection).
    struct PairOps { v4i a0, a1; uint2 da, dw; };
    const auto fetch = [&](int t, int pr, PairOps& o) {
        const int b = 2 * pr;
        o.a0 = lds_a[b * 64 + lane];
        o.a1 = lds_a[(b + 1) * 64 + lane];
        o.da = lds_d[b * 32 + lane];                   // lanes 0..31: rows of block b, 32..63: of block b + 1
        o.dw = uint2{my_wd[(t * (NBLK / 2) + pr) * 64], 0u};
    };
    PairOps ops_even, ops_odd;                          // pairs take them in turn, by name
    fetch(0, 0, ops_even);
#pragma unroll
    for (int t = 0; t < CPW; ++t) {
        // one basic block per column tile (see opaque_one()), and scheduling fences between the pairs inside
        // it: left alone, the compiler issues every MFMA of the unrolled code up front and keeps all of
        // their results alive at once
        if (!opaque_one()) continue;
        const int ct = wave + t * NW;
        if (ct >= mct) break;                          // wave-uniform
        const int m = ct * 32 + j;                     // this lane's output feature
        float acc[RV];
#pragma unroll
        for (int pr = 0; pr < NBLK / 2; ++pr) {
            // a basic block per pair: instruction selection orders a block's pure arithmetic as it likes, and
            // under register pressure it has put every MFMA first and spilled their results
            if (!opaque_one()) continue;
            const int b = 2 * pr;
            const int q = t * (NBLK / 2) + pr;          // pairs in the order they are taken
            PairOps& cur = (q & 1) ? ops_odd : ops_even;
            PairOps& nxt = (q & 1) ? ops_even : ops_odd;
            if (pr + 1 < NBLK / 2) fetch(t, pr + 1, nxt);
            else if (t + 1 < CPW) fetch(t + 1, 0, nxt);
            // both block sums and the scale tables at once; the settlements follow as their operands complete
            v16i zero_i;
#pragma unroll
            for (int r = 0; r < 16; ++r) zero_i[r] = 0;
            v16i s0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(cur.a0, wq[t][b], zero_i, 0, 0, 0);
            v32f scl = __builtin_amdgcn_mfma_f32_32x32x4f16(__builtin_bit_cast(v4h, cur.da), __builtin_bit_cast(v4h, cur.dw), zero_f, 0, 0, 0);
            v16i s1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(cur.a1, wq[t][b + 1], zero_i, 0, 0, 0);
            // all three are issued before the first settlement: the empty statement needs their results, and
            // instruction selection, which places pure arithmetic where it likes, cannot move it
            asm volatile("" : "+v"(s0), "+v"(scl), "+v"(s1));
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int r = 0; r < RV; ++r) acc[r] = __builtin_fmaf(static_cast<float>(s0[r]), scl[r], pr == 0 ? 0.0f : acc[r]);
#pragma unroll
            for (int r = 0; r < RV; ++r) acc[r] = __builtin_fmaf(static_cast<float>(s1[r]), scl[16 + r], acc[r]);
            if (DUMP && sums_dump) {
#pragma unroll
                for (int r = 0; r < RV; ++r) {
                    const int tok = tok0 + mfma32_row(r, lane);
                    if (tok < N && m < M) {
                        sums_dump[(static_cast<int64_t>(tok) * M + m) * NBLK + b] = static_cast<int>(s0[r]);
                        sums_dump[(static_cast<int64_t>(tok) * M + m) * NBLK + b + 1] = static_cast<int>(s1[r]);
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // each half-wave writes one full 128-byte line of a C row per register
        if (m < M) {
#pragma unroll
            for (int r = 0; r < RV; ++r) {
                const int tok = tok0 + mfma32_row(r, lane);
                if (tok < N) __builtin_nontemporal_store(acc[r], C + static_cast<int64_t>(tok) * M + m);
            }
        }
    }
}

template <int TOK, int NBLK, int CPW, bool DUMP, bool Q81>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3))) void q8_linear_ll_kernel(
    const uint8_t* __restrict__ W, const float* __restrict__ X, float* __restrict__ C,
    int M, int N, int relu, uint8_t* __restrict__ xq_dump, int32_t* __restrict__ sums_dump) {
    q8_linear_ll_body<TOK, NBLK, CPW, DUMP, Q81>(W, X, C, M, N, relu, xq_dump, sums_dump);
}
template <int TOK, int NBLK, int CPW, bool DUMP, bool Q81>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void q8_linear_ll2_kernel(
    const uint8_t* __restrict__ W, const float* __restrict__ X, float* __restrict__ C,
    int M, int N, int relu, uint8_t* __restrict__ xq_dump, int32_t* __restrict__ sums_dump) {
    q8_linear_ll_body<TOK, NBLK, CPW, DUMP, Q81>(W, X, C, M, N, relu, xq_dump, sums_dump);
}

template <int TOK, int NBLK, int CPW, bool Q81>
int launch_q8_linear_ll(const void* W, const float* X, float* C, int M, int N, int relu,
                        void* xq_dump, int32_t* sums_dump, hipStream_t stream) {
    const dim3 grid((N + TOK - 1) / TOK), block(256);
    if constexpr (TOK == 32) {
        if (xq_dump || sums_dump)
            hipLaunchKernelGGL((q8_linear_ll2_kernel<TOK, NBLK, CPW, true, Q81>), grid, block, 0, stream, static_cast<const uint8_t*>(W), X, C,
                               M, N, relu, static_cast<uint8_t*>(xq_dump), sums_dump);
        else
            hipLaunchKernelGGL((q8_linear_ll2_kernel<TOK, NBLK, CPW, false, Q81>), grid, block, 0, stream, static_cast<const uint8_t*>(W), X, C,
                               M, N, relu, static_cast<uint8_t*>(nullptr), static_cast<int32_t*>(nullptr));
    } else if (xq_dump || sums_dump)
        hipLaunchKernelGGL((q8_linear_ll_kernel<TOK, NBLK, CPW, true, Q81>), grid, block, 0, stream, static_cast<const uint8_t*>(W), X, C,
                           M, N, relu, static_cast<uint8_t*>(xq_dump), sums_dump);
    else
        hipLaunchKernelGGL((q8_linear_ll_kernel<TOK, NBLK, CPW, false, Q81>), grid, block, 0, stream, static_cast<const uint8_t*>(W), X, C,
                           M, N, relu, static_cast<uint8_t*>(nullptr), static_cast<int32_t*>(nullptr));
    return check_launch("q8_linear_ll_kernel");
}

// Shape gate of the low-latency kernel; returns -1 when the weight-stationary kernel (or the general one)
// should take the call.  `force` = 8 or 16 picks that unit size whatever the gate says (measurements).
template <bool Q81>
int try_q8_linear_ll(const void* W, const float* X, float* C, int M, int N, int nblk, int c_trans,
                     int relu, int force, void* xq_dump, int32_t* sums_dump, hipStream_t stream) {
    if (!c_trans) return -1;
    const int mct = (M + 31) / 32;
    const int cpw = nblk == 16 ? 1 : nblk == 8 ? 2 : nblk == 4 ? 4 : 0;
    if (cpw == 0 || mct > 4 * cpw) return -1;          // the wave's share of the weight must fit 64 registers
    int tok = force;
    if (tok == 0) {
        // Measured crossover against the weight-stationary kernel (us, low-latency / weight-stationary):
        //   408 x 256 -> 256   4.4 (TOK 8) / 5.2       2601 x 128 -> 128   4.3 (16) / 5.1      2601 x 256 -> 256  5.5 (16) / 5.6
        //   10609 x 512 -> 128 10.2 (16) / 12.4        10609 x 128 -> 512  7.9 (16) / 7.1      26368 x 256 -> 768  no instance / 24
        // i.e. it wins while all its work-groups are resident at once (three per CU) and the output is narrow.
        const int resident = 3 * device_cu_count();
        if (N <= 2048) tok = 8;
        else if (N <= 4096 || (nblk == 16 && (N + 15) / 16 <= resident)) tok = 16;
        // K = 512 beyond that, while units of 32 tokens are all resident at two work-groups per CU (they need the
        // registers of two waves per SIMD): 16000 x 512 -> 128 11.2 us against 12.0 weight-stationary (at 10609 rows,
        // where units of 16 are all resident, 10.6 against their 9.7)
        else if (nblk == 16 && (N + 31) / 32 <= 2 * device_cu_count()) tok = 32;
        else return -1;
    }
#define PPML_LL(TOK, NBLK, CPW) if (tok == TOK && nblk == NBLK) return launch_q8_linear_ll<TOK, NBLK, CPW, Q81>(W, X, C, M, N, relu, xq_dump, sums_dump, stream)
    PPML_LL(8, 4, 4);  PPML_LL(8, 8, 2);  PPML_LL(8, 16, 1);
    PPML_LL(16, 4, 4); PPML_LL(16, 8, 2); PPML_LL(16, 16, 1);
    PPML_LL(32, 16, 1);
#undef PPML_LL
    return -1;
}

template <int WT>
int dispatch_q8_linear(const void* W, const float* X, float* C, int M, int N, int nblk, int c_trans,
                       int relu, void* xq_dump, int32_t* sums_dump, hipStream_t stream) {
    // four waves share a token tile; with at most two pairs of column tiles two waves are enough
    if (M <= 128) return launch_q8_linear<2, WT>(W, X, C, M, N, nblk, c_trans, relu, xq_dump, sums_dump, stream);
    return launch_q8_linear<4, WT>(W, X, C, M, N, nblk, c_trans, relu, xq_dump, sums_dump, stream);
}

}  // namespace
}  // namespace ppmlhip

using namespace ppmlhip;

extern "C" int quantize_rows_q8_0_hip(const float* x, void* y, int64_t ne, ppml_hip_stream_t stream) {
    if (!x || !y || ne <= 0 || (ne % QK) != 0) { set_error("quantize_rows_q8_0_hip: bad arguments (ne=%lld)", (long long)ne); return RC_BAD_ARGS; }
    const int64_t nblocks = ne / QK;
    const int64_t threads = nblocks * 4;
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

extern "C" int quantize_rows_q8_1_hip(const float* x, void* y, int64_t ne, ppml_hip_stream_t stream) {
    if (!x || !y || ne <= 0 || (ne % QK) != 0) { set_error("quantize_rows_q8_1_hip: bad arguments (ne=%lld)", (long long)ne); return RC_BAD_ARGS; }
    const int64_t nblocks = ne / QK;
    const unsigned grid = static_cast<unsigned>((nblocks * 4 + 255) / 256);
    hipLaunchKernelGGL(quantize_rows_q8_1_kernel, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream),
                       x, static_cast<uint8_t*>(y), nblocks);
    return check_launch("quantize_rows_q8_1_kernel") ? RC_BAD_ARGS : RC_OK;   // reference launcher: 0 / 1
}

extern "C" int dequantize_q8_1_hip(const void* x, float* y, int64_t ne, ppml_hip_stream_t stream) {
    if (!x || !y || ne <= 0) { set_error("dequantize_q8_1_hip: bad arguments"); return RC_BAD_ARGS; }
    const unsigned grid = static_cast<unsigned>((ne + 255) / 256);
    hipLaunchKernelGGL(dequantize_q8_1_kernel, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint8_t*>(x), y, ne);
    return check_launch("dequantize_q8_1_kernel") ? RC_BAD_ARGS : RC_OK;
}

extern "C" size_t q8_weight_packed_bytes_hip(int M, int K);
extern "C" int q8_weight_pack_hip(const void* W, int wtype, int M, int K, void* packed, ppml_hip_stream_t stream);

namespace ppmlhip {
namespace {

// ------------------------------------------------------------------------------------------
// Tiled form of the same linear, for Q8_0M weights too large for the weight-stationary kernel under many
// tokens (K from 1024 on, or more columns than its instances hold).  The general kernel gives a work-group 32
// tokens and streams the WHOLE weight through it: 4096 tokens x 4096 -> 4096 reads the 16 MB weight 128 times
// (900 us, 0.03 of the int8 matrix peak).  Here the problem is cut like a GEMM:
//
//   1. the activations are quantized once, into a workspace, in the layout the packed weight has: per tile of
//      32 tokens and block of 32 k the 64 lanes' sixteen quants (1 KB, an MFMA operand as it lies), and a plane
//      of fp16 scales [tile][block][32] (q8_quantize_fragments_kernel: the arithmetic of quantize_block_lane,
//      tokens past the end quantize zeros);
//   2. q8_tiled_kernel: one work-group of eight waves per 128 tokens x 256 features; wave (wr, wc) owns 64 x 64
//      of it (2 x 2 accumulator tiles) -- or, where that leaves CUs without work or in a thin last round, per 128 x
//      128, a wave 64 x 32 (the launcher's rule).  K is walked in stages of two blocks: every thread copies sixteen
//      bytes of activation fragments and thirty-two of weight fragments (plus the scales) from memory to the
//      other half of a double buffer in LDS -- requested one stage ahead, into registers --, one barrier per
//      stage.  Per stage and accumulator tile: two v_mfma_i32_32x32x32_i8 that start from 1.5 * 2^23 (exact
//      block sums, read as floats), two v_mfma_f32_32x32x8_bf16 that take the offset off, one
//      v_mfma_f32_32x32x4_2b_f16 for the two scale tables d_a[token] * d_w[feature] (each entry the exact
//      product of two halves), and 2 x 16 fma on the vector pipe:
//          acc = fma(float(sumi), d_w * d_a, acc)        blocks ascending
//      -- the settlement of every other kernel of this file: same bits.
//
// c_trans = 0 (C [M][N]) swaps the operands of the MFMAs, as the weight-stationary kernel does.
// ------------------------------------------------------------------------------------------
constexpr int QT_TOK_TILES = 4;                            // a work-group's tile in units of 32: 128 tokens x (128 TJ) features,
template <int TJ> struct QTile {                           // TJ = column tiles per wave (2: the wide form, 1: the narrow one)
    static constexpr int COL_TILES = 4 * TJ;
    static constexpr int A = QT_TOK_TILES * 2 * 1024;      // a stage: activation fragments [token tile][block of the pair][1 KB]
    static constexpr int W = COL_TILES * 2 * 1024;         //          weight fragments [column tile][block][1 KB]
    static constexpr int DA = QT_TOK_TILES * 2 * 32 * 2;   //          activation scales [token tile][block][32] fp16
    static constexpr int DW = COL_TILES * 2 * 32 * 2;      //          weight scales [column tile][block][32] fp16
    static constexpr int STAGE = A + W + DA + DW;
};
constexpr uint32_t QT_OUTSIDE = 0x80000000u;               // an offset no buffer of this kernel reaches

// One wave per (token tile, its upper or lower sixteen tokens, block): four lanes hold a block in element order.
template <bool Q81>
__global__ __launch_bounds__(256) void q8_quantize_fragments_kernel(const float* __restrict__ X, uint8_t* __restrict__ xq,
                                                                    uint16_t* __restrict__ xd, int N, int nblk, int relu, int total_waves) {
    const int lane = threadIdx.x & 63;
    const int gw = __builtin_amdgcn_readfirstlane(static_cast<int>(blockIdx.x) * 4 + static_cast<int>(threadIdx.x >> 6));
    if (gw >= total_waves) return;                      // wave-uniform
    const int b = gw % nblk, rest = gw / nblk;
    const int half = rest & 1, tile = rest >> 1;
    const int c4 = lane & 3, r = half * 16 + (lane >> 2);
    const int row = tile * 32 + r;
    v4f x0 = {0.f, 0.f, 0.f, 0.f}, x1 = {0.f, 0.f, 0.f, 0.f};
    if (row < N) {
        const float* src = X + (static_cast<int64_t>(row) * nblk + b) * QK + c4 * 8;
        x0 = *reinterpret_cast<const v4f_u*>(src);
        x1 = *reinterpret_cast<const v4f_u*>(src + 4);
    }
    const BlockQuant bq = (relu & 1) ? quantize_block_lane<Q81, true>(x0, x1) : quantize_block_lane<Q81, false>(x0, x1);
    const size_t frag = static_cast<size_t>(tile) * nblk + b;
    *reinterpret_cast<uint2*>(xq + (frag << 10) + (((c4 >> 1) * 32 + r) << 4) + ((c4 & 1) << 3)) = uint2{bq.q_lo, bq.q_hi};
    if (c4 == 0) xd[frag * 32 + r] = bq.d_bits;
}

template <bool CT0, int TJ>
__global__ __launch_bounds__(512) void q8_tiled_kernel(const uint8_t* __restrict__ xq, const uint16_t* __restrict__ xd,
                                                       const uint8_t* __restrict__ W, float* __restrict__ C, int M, int N, int nblk,
                                                       int ntt_pad, int mct_pad, int tiles_t, int tiles_c) {
    using T = QTile<TJ>;
    __shared__ __attribute__((aligned(16))) uint8_t lds[2][T::STAGE];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 31, hh = lane >> 5;
    const int wr = wave >> 2, wc = wave & 3;

    // work-group -> tile: bands of eight token tiles, the column tiles of a band side by side in one XCD's L2
    int tile_t, tile_c;
    {
        int t = xcd_contiguous_index(static_cast<int>(blockIdx.x), tiles_t * tiles_c);
        const int band_rows = 8;
        const int band = t / (band_rows * tiles_c);
        t -= band * band_rows * tiles_c;
        const int rows_here = (tiles_t - band * band_rows) < band_rows ? (tiles_t - band * band_rows) : band_rows;
        tile_t = band * band_rows + t % rows_here;
        tile_c = t / rows_here;
    }
    const int tt0 = tile_t * QT_TOK_TILES, ct0 = tile_c * T::COL_TILES;
    const int stages = nblk / 2;

    const __amdgpu_buffer_rsrc_t rsrc_xq = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(xq), 0, ntt_pad * nblk * 1024, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_xd = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(xd), 0, ntt_pad * nblk * 64, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_wq = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(W), 0, mct_pad * nblk * 1024, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_wd = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(W) + static_cast<size_t>(mct_pad) * nblk * 1024, 0,
                                                                             mct_pad * nblk * 64, 0x00020000);
    // this thread's shares of a stage (the two blocks of a pair lie side by side in memory: 2 KB of fragments, 128
    // bytes of scales per tile).  Column tiles past the weight's padded end repeat the last one; never stored.
    const auto col_tile = [&](int c) { return c < mct_pad ? c : mct_pad - 1; };
    uint32_t a_off = static_cast<uint32_t>((tt0 + (tid >> 7)) * nblk) * 1024u + static_cast<uint32_t>(tid & 127) * 16u;
    uint32_t w_off[TJ];
#pragma unroll
    for (int i = 0; i < TJ; ++i) w_off[i] = static_cast<uint32_t>(col_tile(ct0 + (tid >> 7) + 4 * i) * nblk) * 1024u + static_cast<uint32_t>(tid & 127) * 16u;
    // scales: threads 0..31 the activations' (four tiles x 128 bytes), threads 64 .. 63 + 32 TJ the weight's (128 bytes
    // per column tile); the others request nothing (an offset outside), so every wave counts the same loads
    const bool dw_thread = tid >= 64 && tid < 64 + 32 * TJ;
    uint32_t da_off = tid < 32 ? static_cast<uint32_t>((tt0 + (tid >> 3)) * nblk) * 64u + static_cast<uint32_t>(tid & 7) * 16u : QT_OUTSIDE;
    uint32_t dw_off = dw_thread ? static_cast<uint32_t>(col_tile(ct0 + ((tid - 64) >> 3)) * nblk) * 64u + static_cast<uint32_t>(tid & 7) * 16u
                                               : QT_OUTSIDE;
    v4i ra, rw[TJ], rda, rdw;
    const auto request = [&](int s) {                   // (s past the last stage: outside, zeros)
        const uint32_t fo = static_cast<uint32_t>(s) * 2048u, so = static_cast<uint32_t>(s) * 128u;
        const bool live = s < stages;
        ra = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_xq, live ? a_off + fo : QT_OUTSIDE, 0, 0));
#pragma unroll
        for (int i = 0; i < TJ; ++i) rw[i] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_wq, live ? w_off[i] + fo : QT_OUTSIDE, 0, 0));
        rda = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_xd, (live && tid < 32) ? da_off + so : QT_OUTSIDE, 0, 0));
        rdw = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_wd, (live && dw_thread) ? dw_off + so : QT_OUTSIDE, 0, 0));
    };
    const auto deposit = [&](uint8_t* stage) {
        *reinterpret_cast<v4i*>(stage + tid * 16) = ra;
#pragma unroll
        for (int i = 0; i < TJ; ++i) *reinterpret_cast<v4i*>(stage + T::A + (tid + 512 * i) * 16) = rw[i];
        if (tid < 32) *reinterpret_cast<v4i*>(stage + T::A + T::W + tid * 16) = rda;
        if (dw_thread) *reinterpret_cast<v4i*>(stage + T::A + T::W + T::DA + (tid - 64) * 16) = rdw;
    };

    // (see the weight-stationary kernel: block sums leave the matrix pipe as floats)
    v16i magic_i;
#pragma unroll
    for (int r = 0; r < 16; ++r) magic_i[r] = WS_MAGIC_BITS;
    asm volatile("" : "+v"(magic_i));
    typedef short v4s __attribute__((ext_vector_type(4)));
    typedef _Float16 v4h __attribute__((ext_vector_type(4)));
    v4s unbias_a = {static_cast<short>(0xCAC0), 0, 0, 0};   // bf16 -0.75 * 2^23
    v4s unbias_b = {static_cast<short>(0x3F80), 0, 0, 0};   // bf16 1
    asm volatile("" : "+v"(unbias_a), "+v"(unbias_b));
    v32f zero_f2;
#pragma unroll
    for (int r = 0; r < 32; ++r) zero_f2[r] = 0.0f;

    v16f acc[2][TJ];
#pragma unroll
    for (int ti = 0; ti < 2; ++ti)
#pragma unroll
        for (int tj = 0; tj < TJ; ++tj)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[ti][tj][r] = 0.0f;

    request(0);
    for (int s = 0; s < stages; ++s) {
        uint8_t* stage = lds[s & 1];
        deposit(stage);
        request(s + 1);
        __syncthreads();                                // stage s is in LDS; every wave has left stage s - 1
        // this wave's operands of the stage: fragments a[token tile][block], w[column tile][block]; scales da / dw: lanes
        // 0..31 hold the rows (columns) of the pair's first block, lanes 32..63 of its second, the scale in the first of a
        // lane's four k slots, zeros in the others
        v4i a[2][2], w[TJ][2];
        uint2 da[2], dw[TJ];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int blk = 0; blk < 2; ++blk) a[t][blk] = *reinterpret_cast<const v4i*>(stage + (((2 * wr + t) * 2 + blk) << 10) + lane * 16);
            da[t] = uint2{*reinterpret_cast<const uint16_t*>(stage + T::A + T::W + ((2 * wr + t) * 2 + hh) * 64 + j * 2), 0u};
        }
#pragma unroll
        for (int t = 0; t < TJ; ++t) {
#pragma unroll
            for (int blk = 0; blk < 2; ++blk) w[t][blk] = *reinterpret_cast<const v4i*>(stage + T::A + (((TJ * wc + t) * 2 + blk) << 10) + lane * 16);
            dw[t] = uint2{*reinterpret_cast<const uint16_t*>(stage + T::A + T::W + T::DA + ((TJ * wc + t) * 2 + hh) * 64 + j * 2), 0u};
        }
        // accumulator tile c of the wave: token tile c / TJ, column tile c % TJ
        const auto block_sum = [&](int c, int blk) {
            const int ti = c / TJ, tj = c % TJ;
            if constexpr (CT0) return __builtin_amdgcn_mfma_i32_32x32x32_i8(w[tj][blk], a[ti][blk], magic_i, 0, 0, 0);
            else return __builtin_amdgcn_mfma_i32_32x32x32_i8(a[ti][blk], w[tj][blk], magic_i, 0, 0, 0);
        };
        const auto to_float = [&](const v16i& biased) {     // 1.5 * 2^23 + sum -> float(sum), on the matrix pipe
            return __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(unbias_a, unbias_b, __builtin_bit_cast(v16f, biased), 0, 0, 0);
        };
        const auto scale_tables = [&](int c) {             // d_a[token] * d_w[feature] of both blocks of tile c
            const int ti = c / TJ, tj = c % TJ;
            if constexpr (CT0) return __builtin_amdgcn_mfma_f32_32x32x4f16(__builtin_bit_cast(v4h, dw[tj]), __builtin_bit_cast(v4h, da[ti]), zero_f2, 0, 0, 0);
            else return __builtin_amdgcn_mfma_f32_32x32x4f16(__builtin_bit_cast(v4h, da[ti]), __builtin_bit_cast(v4h, dw[tj]), zero_f2, 0, 0, 0);
        };
        // The stage's 4 TJ units (accumulator tile u / 2, block u % 2) with the matrix pipe ahead of the vector pipe, the
        // order of the weight-stationary kernel's steps; the barriers keep the compiler from sinking every MFMA next to
        // its consumer, where each settlement would wait out a whole MFMA.  The wide form, with 64 accumulator registers,
        // has room for two buffers of block sums: while unit u is settled, the block sum of unit u + 1 runs, and the
        // offset comes off it right in front of its settlement.  The narrow form has room for three: the matrix pipe is
        // two units ahead, and a settlement reads nothing that was issued less than a whole unit ago.  (Neither makes the
        // two pipes overlap: their times add up in both.)
        constexpr int UNITS = 4 * TJ, DEPTH = TJ == 2 ? 1 : 2;
        v16i sum[DEPTH + 1];
        v16f flt[DEPTH + 1];
        v32f scl[2];                                       // the tables of a tile and of the next one, taking turns by name
        sum[0] = block_sum(0, 0);
        scl[0] = scale_tables(0);
        if constexpr (DEPTH == 2) {
            sum[1] = block_sum(0, 1);
            flt[0] = to_float(sum[0]);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < UNITS; ++u) {
            const int c = u >> 1, ti = c / TJ, tj = c % TJ;
            if constexpr (DEPTH == 1) {
                flt[u & 1] = to_float(sum[u & 1]);
                if (u + 1 < UNITS) {
                    sum[(u + 1) & 1] = block_sum((u + 1) >> 1, (u + 1) & 1);
                    if (((u + 1) & 1) == 0) scl[((u + 1) >> 1) & 1] = scale_tables((u + 1) >> 1);
                }
            } else {
                if (u + 2 < UNITS) {
                    sum[(u + 2) % 3] = block_sum((u + 2) >> 1, (u + 2) & 1);
                    if (((u + 2) & 1) == 0) scl[((u + 2) >> 1) & 1] = scale_tables((u + 2) >> 1);
                }
                if (u + 1 < UNITS) flt[(u + 1) % 3] = to_float(sum[(u + 1) % 3]);
            }
            __builtin_amdgcn_sched_barrier(0);
            const v16f& f = flt[u % (DEPTH + 1)];
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[ti][tj][r] = __builtin_fmaf(f[r], scl[c & 1][(u & 1) * 16 + r], acc[ti][tj][r]);
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // the finished tile: a half-wave store is one 128-byte run of a C row; what lies outside C is dropped by the buffer
    // (rows past the end lie behind it, columns past the end start from 2^31: the launcher keeps C below that)
    const __amdgpu_buffer_rsrc_t rsrc_c = __builtin_amdgcn_make_buffer_rsrc(C, 0, static_cast<int>(static_cast<int64_t>(M) * N * 4), 0x00020000);
#pragma unroll
    for (int ti = 0; ti < 2; ++ti) {
#pragma unroll
        for (int tj = 0; tj < TJ; ++tj) {
            const int tok0 = (tt0 + 2 * wr + ti) * 32, m0 = (ct0 + TJ * wc + tj) * 32;
            uint32_t off;
            int pitch;
            if constexpr (CT0) {       // rows of C are features, the lane's token picks the column
                off = (tok0 + j < N && m0 < mct_pad * 32) ? (static_cast<uint32_t>(m0 + 4 * hh) * N + (tok0 + j)) * 4u : QT_OUTSIDE;
                pitch = N * 4;
            } else {
                off = m0 + j < M ? (static_cast<uint32_t>(tok0 + 4 * hh) * M + (m0 + j)) * 4u : QT_OUTSIDE;
                pitch = M * 4;
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(acc[ti][tj][r]), rsrc_c, off, 0, WS_STORE_AUX);
                off += ((r & 3) == 3 ? 5 : 1) * pitch;  // rows 8 * (r / 4) + r % 4 (+ 4 in the upper half-wave)
            }
        }
    }
}

// -1: not a problem for this form, or no workspace to be had (the caller goes on to the general kernel)
// `wtype` other than PPML_WTYPE_Q8_0M: the weight is packed into the workspace first, per call (one pass over it: 4096 x
// 4096 in 10 us, against the 700 us that the general kernel loses on such a weight).
template <bool Q81>
int try_q8_tiled(const void* W, int wtype, const float* X, float* C, int M, int N, int nblk, int c_trans, int relu, hipStream_t stream) {
    if (nblk % 2 != 0) return -1;                       // stages are pairs of blocks
    const int ntt = (N + 31) / 32, ntt_pad = (ntt + QT_TOK_TILES - 1) / QT_TOK_TILES * QT_TOK_TILES;
    const int mct = (M + 31) / 32, mct_pad = packed_tiles(M);
    const int tiles_t = ntt_pad / QT_TOK_TILES;
    // The form: tiles 256 features wide (two column tiles per wave) or 128 wide (one).  A CU holds one work-group of
    // either; a wide one takes 1.8 times as long as a narrow one for twice the outputs, so the form with the cheaper
    // rounds wins: us, wide / narrow, with the work-groups of each: 4096 x 4096 -> 4096  199 / 222 (512, 1024), 8192 x
    // 1024 -> 8192  216 / 233, 16384 x 512 -> 4096  118 / 131, 5000 x 2048 -> 1000  55 / 60 (160, 320), 26368 x 1024 ->
    // 256  44 / 47 (206, 412); 408 x 4096 -> 4096  80 / 51 (64, 128), 2048 x 1024 -> 1024  26 / 19, 512 x 1024 -> 1024
    // 24 / 16, 2601 x 1024 -> 512  26 / 19, 10609 x 1024 -> 128  31 / 23, 10609 x 512 -> 1024  35 / 32 (332, 664),
    // 26368 x 512 -> 1024  65 / 63.
    const int cus = device_cu_count();
    const int64_t wgs_wide = static_cast<int64_t>(tiles_t) * ((mct + 7) / 8), wgs_narrow = static_cast<int64_t>(tiles_t) * ((mct + 3) / 4);
    const bool narrow = static_cast<double>((wgs_narrow + cus - 1) / cus) < 1.8 * static_cast<double>((wgs_wide + cus - 1) / cus);
    const int ctiles = narrow ? 4 : 8;
    const int tiles_c = (mct + ctiles - 1) / ctiles;
    // Where it pays at all: from sixteen work-groups on (a work-group walks the whole K by itself), at least half a
    // narrow tile of features.  us, general kernel / this one: 4096 x 4096 -> 4096  900 / 199, 408 x 4096 -> 4096  905 /
    // 51, 128 x 1024 -> 4096  199 / 15, 2048 x 1024 -> 1024  52 / 19, 1024 x 1024 -> 256  19 / 16, 26368 x 1024 -> 1024
    // 116 / 108.
    if (M < 64 || static_cast<int64_t>(tiles_t) * tiles_c < 16) return -1;
    // 32-bit byte offsets everywhere: the fragments of both operands and C with the rows of its last, ragged tile
    const int64_t xq_bytes = static_cast<int64_t>(ntt_pad) * nblk * 1024, xd_bytes = static_cast<int64_t>(ntt_pad) * nblk * 64;
    const int64_t wq_bytes = static_cast<int64_t>(mct_pad) * nblk * 1024;
    const int64_t c_reach = c_trans ? static_cast<int64_t>(ntt_pad * 32 + 4) * M * 4 : static_cast<int64_t>(tiles_c * ctiles * 32 + 4) * N * 4;
    if (xq_bytes >= 0x7fff0000LL || wq_bytes >= 0x7fff0000LL || c_reach >= 0x7fff0000LL) return -1;
    if (static_cast<int64_t>(tiles_t) * tiles_c > 0x7fffffffLL) return -1;
    const size_t wp_bytes = wtype == PPML_WTYPE_Q8_0M ? 0 : (q8_weight_packed_bytes_hip(M, nblk * QK) + 1023) / 1024 * 1024;
    const Workspace held = workspace_take(static_cast<size_t>(xq_bytes + xd_bytes) + wp_bytes, stream);
    if (!held.ptr) return -1;
    uint8_t* xq = held.ptr;
    uint16_t* xd = reinterpret_cast<uint16_t*>(held.ptr + xq_bytes);
    int rc = RC_OK;
    if (wp_bytes) {
        uint8_t* wp = held.ptr + xq_bytes + xd_bytes;
        rc = q8_weight_pack_hip(W, wtype, M, nblk * QK, wp, stream);
        W = wp;
    }
    const int total_waves = ntt_pad * 2 * nblk;
    if (rc == RC_OK) {
        hipLaunchKernelGGL((q8_quantize_fragments_kernel<Q81>), dim3((total_waves + 3) / 4), dim3(256), 0, stream, X, xq, xd, N, nblk, relu, total_waves);
        rc = check_launch("q8_quantize_fragments_kernel");
    }
    if (rc == RC_OK) {
        const dim3 grid(static_cast<unsigned>(tiles_t * tiles_c)), block(512);
#define PPML_QT(CT0_, TJ_) hipLaunchKernelGGL((q8_tiled_kernel<CT0_, TJ_>), grid, block, 0, stream, xq, xd, static_cast<const uint8_t*>(W), C, M, N, nblk, \
                                              ntt_pad, mct_pad, tiles_t, tiles_c)
        if (narrow) { if (c_trans) PPML_QT(false, 1); else PPML_QT(true, 1); }
        else        { if (c_trans) PPML_QT(false, 2); else PPML_QT(true, 2); }
#undef PPML_QT
        rc = check_launch("q8_tiled_kernel");
    }
    workspace_give(held, stream);
    return rc;
}

}  // namespace
}  // namespace ppmlhip

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
    const int relu = flags & 1;                        // bit 0: ReLU on X
    const int act = flags & 3;                         // bit 1: Q8_1 rule for the activations
    hipStream_t s = static_cast<hipStream_t>(stream);
    StatsScope stat("hip/q8-general", M, K, N, s);
    set_q8_path(PPML_Q8_PATH_GENERAL);
    // the kernel families that want the packed layout and keep the weight resident or close by; -1: none of them ran
    const auto resident_families = [&](const void* Wp) -> int {
        const int ll_bits = flags & (PPML_Q8_FLAG_LOW_LATENCY_8 | PPML_Q8_FLAG_LOW_LATENCY_16);
        const int force_ll = ll_bits == PPML_Q8_FLAG_LOW_LATENCY_32 ? 32 : ll_bits == PPML_Q8_FLAG_LOW_LATENCY_8 ? 8 :
                             ll_bits == PPML_Q8_FLAG_LOW_LATENCY_16 ? 16 : 0;
        const int rl = (flags & PPML_Q8_FLAG_NO_LOW_LATENCY) ? -1
                     : (act & 2) ? try_q8_linear_ll<true>(Wp, X, C, M, N, nblk, c_trans, relu, force_ll, xq_dump, sums_dump, s)
                                 : try_q8_linear_ll<false>(Wp, X, C, M, N, nblk, c_trans, relu, force_ll, xq_dump, sums_dump, s);
        if (rl >= 0) { set_q8_path(PPML_Q8_PATH_LOW_LATENCY); stat.set_path("hip/q8-low-latency"); return rl; }
        const int csplit = (flags & PPML_Q8_FLAG_COLUMN_PARTS) ? 1 : (flags & PPML_Q8_FLAG_NO_COLUMN_PARTS) ? -1 : 0;
        const int rc = (flags & PPML_Q8_FLAG_NO_WEIGHT_STATIONARY) ? -1
                     : (act & 2) ? try_q8_linear_ws<true>(Wp, X, C, M, N, nblk, c_trans, relu, csplit, xq_dump, sums_dump, s)
                                 : try_q8_linear_ws<false>(Wp, X, C, M, N, nblk, c_trans, relu, csplit, xq_dump, sums_dump, s);
        if (rc >= 0) { set_q8_path(PPML_Q8_PATH_WEIGHT_STATIONARY); stat.set_path("hip/q8-weight-stationary"); return rc; }
        return -1;
    };
    // (the diagnostic buffers are the general kernel's; PPML_Q8_FLAG_NO_TILED keeps a call there too)
    const auto tiled = [&]() -> int {
        const int rt = ((flags & PPML_Q8_FLAG_NO_TILED) || xq_dump || sums_dump) ? -1
                     : (act & 2) ? try_q8_tiled<true>(W, wtype, X, C, M, N, nblk, c_trans, relu, s)
                                 : try_q8_tiled<false>(W, wtype, X, C, M, N, nblk, c_trans, relu, s);
        if (rt >= 0) { set_q8_path(PPML_Q8_PATH_TILED); stat.set_path("hip/q8-tiled"); }
        return rt;
    };
    // A weight in one of the reference's own layouts (include/ppml/QuantBlocks.h:33-41, 123-133) need not wait for its
    // owner to adopt the packed one.  Beyond what stays resident it takes the tiled kernel, which packs it into its
    // workspace on the way.  Up to that size it is packed into the stream's workspace here (one launch: 3.7 us more
    // than the call on a packed weight) and served by the kernels of the packed layout, wherever that launch costs less
    // than the general kernel loses: from 2^27 products on, and for weights of 64 Ki elements with K >= 512 or 768
    // features whatever the token count.  us on a Q8_0 weight, general kernel / this way: 26368 x 256 -> 768  60 / 22.9
    // (20.8 on a weight packed at load), 26368 x 256 -> 256  26.8 / 12.3, 105472 x 64 -> 256  39.6 / 21.9, 10609 x 64 ->
    // 256  8.1 / 7.1, 2601 x 256 -> 256  8.4 / 7.0, 64 x 512 -> 128  14.0 / 7.8, 128 x 256 -> 768  16.7 / 9.8; below the
    // rule: 5000 x 64 -> 256  5.5 / 6.9, 26368 x 64 -> 64  6.6 / 7.2, 1024 x 128 -> 128  5.6 / 7.8.  No workspace (a stream
    // under capture): the general kernel, as before.
    if (wtype == PPML_WTYPE_Q8_0 || wtype == PPML_WTYPE_Q8_1 || wtype == PPML_WTYPE_Q8_0R) {
        if (static_cast<int64_t>(M) * K > (256 << 10)) {
            const int rt = tiled();
            if (rt >= 0) return rt;
        } else if ((static_cast<int64_t>(N) * M * K >= (1LL << 27) || (static_cast<int64_t>(M) * K >= (64 << 10) && (K >= 512 || M >= 768))) &&
                   !xq_dump && !sums_dump &&
                   (flags & (PPML_Q8_FLAG_NO_LOW_LATENCY | PPML_Q8_FLAG_NO_WEIGHT_STATIONARY)) != (PPML_Q8_FLAG_NO_LOW_LATENCY | PPML_Q8_FLAG_NO_WEIGHT_STATIONARY)) {
            const Workspace held = workspace_take(q8_weight_packed_bytes_hip(M, K), s);
            if (held.ptr) {
                const int rc = q8_weight_pack_hip(W, wtype, M, K, held.ptr, stream) == RC_OK ? resident_families(held.ptr) : -1;
                workspace_give(held, s);
                if (rc >= 0) return rc;
            }
        }
    }
    switch (wtype) {
        case PPML_WTYPE_Q8_0:  return dispatch_q8_linear<PPML_WTYPE_Q8_0>(W, X, C, M, N, nblk, c_trans, act, xq_dump, sums_dump, s);
        case PPML_WTYPE_Q8_1:  return dispatch_q8_linear<PPML_WTYPE_Q8_1>(W, X, C, M, N, nblk, c_trans, act, xq_dump, sums_dump, s);
        case PPML_WTYPE_Q8_0R: return dispatch_q8_linear<PPML_WTYPE_Q8_0R>(W, X, C, M, N, nblk, c_trans, act, xq_dump, sums_dump, s);
        case PPML_WTYPE_Q8_0M: {
            const int rr = resident_families(W);
            if (rr >= 0) return rr;
            const int rt = tiled();
            if (rt >= 0) return rt;
            return dispatch_q8_linear<PPML_WTYPE_Q8_0M>(W, X, C, M, N, nblk, c_trans, act, xq_dump, sums_dump, s);
        }
        default: set_error("mul_mat_q8_hip: unsupported wtype %d", wtype); return RC_WTYPE;
    }
}

// What mul_mat_q8_cuda would report in *path_out for this call (src/cuda/MulMatQ8Kernel.cu:493-496): 1 (its
// MMQ kernels) when PPML_MMQ is not 0 and the token count reaches PPML_MMQ_MIN_N (default 16) or the weight is
// repacked, else 0 (its MMVQ kernels).  Both of its paths give the same numbers and so does this library, whose
// own choice of kernel ppml_hip_q8_last_path() reports; the value is kept for callers that log or count it.
static int reference_path_value(int N, int wtype) {
    const auto env_int = [](const char* name, int fallback) {
        const char* v = std::getenv(name);
        if (!v || !*v) return fallback;
        char* end = nullptr;
        const long x = std::strtol(v, &end, 10);
        return end == v ? fallback : static_cast<int>(x);
    };
    const int min_n = env_int("PPML_MMQ_MIN_N", 16);
    const bool mmq_on = env_int("PPML_MMQ", 1) != 0;
    return (mmq_on && (N >= min_n || wtype == PPML_WTYPE_Q8_0R || wtype == PPML_WTYPE_Q8_0M)) ? 1 : 0;
}

extern "C" int mul_mat_q8_hip(const void* W, const float* X, float* C, int M, int N, int K, int wtype,
                              int c_trans, int* path_out, ppml_hip_stream_t stream) {
    if (path_out) *path_out = 0;
    const int rc = mul_mat_q8_ex_hip(W, X, C, M, N, K, wtype, c_trans, 0, nullptr, nullptr, stream);
    if (rc == RC_OK && path_out) *path_out = reference_path_value(N, wtype);
    return rc;
}
