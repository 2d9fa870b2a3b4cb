// Fused attention forward for gfx950: O = softmax(scale * Q K^T + bias) V in one pass, the twin of the
// reference's flash_attn_forward_cuda (include/ppml/FlashAttn.h:62-65, src/backend/CUDAKernels.cpp:174,
// 894-903) and of its CPU statement flash_attn_forward_cpu (src/ops/FlashAttn.cpp:55-135).  It replaces
// the five-node chain out_prod(K,Q) -> scale -> add bias -> softmax -> out_prod(attn,V) of
// src/modules/Attention.cpp:264-281, whose L x L score planes never reach memory here.
//
// Layout (FlashAttn.h:8-13): Q, K, V, O [B][h][L][d]; bias [B][h][L query][L key]; LSE [B][h][L].
//
// One work-group per (plane, block of 32*NW queries); wave w owns 32 queries.  K and V of the plane
// are staged in LDS (up to CH keys at a time, the whole plane for L <= CH) and shared by the waves.
// The matrix work is arranged so that nothing has to move between lanes:
//
//   scores, transposed:  S^T[key][query] = K_tile (32 keys x d) . Q^T (d x 32 queries)
//       on the bf16 matrix pipe at binary32 accuracy: Q (times scale * log2 e) and K are split into three
//       bf16 parts each (exactly), six partial products per 16 features (see common.hpp); K lies in LDS
//       as ready MFMA fragments, Q in registers.  2.7 times less matrix-pipe time than the fp32 MFMA,
//       which would moreover keep the vector pipe from running beside it;
//       lane (query j = lane % 32, half = lane / 32) ends up with 16 of the 32 keys of ITS query in its
//       accumulator registers -> the softmax row maximum and sum are 16 in-register steps plus one
//       exchange with lane j + 32;
//   output, transposed:  O^T[dd][query] += V^T (d x 32 keys) . P (32 keys x 32 queries)
//       the same arithmetic: the probabilities are split in registers where they were computed, eight
//       score registers making one B operand of 16 keys -- the key order of the contraction is simply
//       the order in which the score registers hold them (key(kk, half) = 8*(kk/4) + 4*half + kk%4) --
//       and V lies in LDS as fragments of V^T in that key order;
//       the running rescale factor alpha and the final 1/(l + eps) are per-lane scalars.
//
#include "common.hpp"

#include <cmath>
#include <type_traits>

namespace ppmlhip {
namespace {

typedef float v2f __attribute__((ext_vector_type(2)));

template <int DP, int NW> struct AttnTiling {
    // keys staged in LDS at a time: 36 KB per four-wave work-group (four of them share a CU and its
    // 160 KB; 128 keys would leave room for three, measured 64.7 against 61.2 us at the MSA shape)
    static constexpr int CH = DP <= 32 ? (NW == 4 ? 96 : 192) : (NW == 4 ? 64 : 128);
    static constexpr int NC = DP / 16;                // 16-feature chunks of the score contraction
    // a 32-key tile of K in LDS: one 1 KB MFMA operand fragment per (chunk, bf16 part), [half][key][8 bf16]
    static constexpr int KT_BYTES = NC * 3 * 1024;
    // a 32-key tile of V in LDS: fragments of V^T per (32 features, 16 keys, bf16 part); slot i of lane
    // (feature, half) holds key 16 ch + 8 (i / 4) + 4 half + i % 4 of the tile
    static constexpr int VT_BYTES = (DP / 32) * 2 * 3 * 1024;
    static constexpr size_t lds_bytes = static_cast<size_t>(CH / 32) * (KT_BYTES + VT_BYTES);
};

struct AttnParams {
    const float* Q; const float* K; const float* V; const float* bias;
    float* O; float* LSE;
    int planes, L, d;
    int causal;
    float scale, eps;
    int head;            // keys of the reference's first block: min(Bc, keys of the row)
    int stage_rows;      // keys staged in LDS at a time: min(CH, L rounded up to 32)
    int in_ld;           // Q, K, V are [B][h][d][L] (the graph's [L, D, h, B] tensors, not yet permuted)
    int out_ld;          // O is written as [B][h][d][L]
};

__device__ __forceinline__ float lane_xor32(float x) {
    // the value of the lane 32 away (same query, other half of the keys)
    return __shfl_xor(x, 32, 64);
}

// PF: request each tile's bias one tile ahead.  It costs 16 registers, i.e. the fourth wave per SIMD, so only
// the instance for short sequences uses it: there a work-group is a chain of memory latencies and the
// machine is far from full anyway.
template <int DP, int NW, bool PF>
// (the instance for long sequences is held to 128 registers: four waves per SIMD)
__global__ __launch_bounds__(NW * 64, (DP <= 32 && !PF) ? 4 : 1) void flash_attn_forward_kernel(const AttnParams p) {
    using T = AttnTiling<DP, NW>;
    constexpr int NC = T::NC, KT_BYTES = T::KT_BYTES, VT_BYTES = T::VT_BYTES;
    constexpr int NB = DP / 32;                       // 32-row blocks of the transposed output
    extern __shared__ __attribute__((aligned(16))) float attn_lds[];
    uint8_t* lds_k = reinterpret_cast<uint8_t*>(attn_lds);
    uint8_t* lds_v = lds_k + (p.stage_rows / 32) * KT_BYTES;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 31, half = lane >> 5;
    const int plane = blockIdx.y;
    const int L = p.L, d = p.d;
    const int q0 = (blockIdx.x * NW + wave) * 32;     // first query of this wave
    const int q = q0 + j;                             // this lane's query
    const bool wave_active = q0 < L;                  // wave-uniform
    const int64_t plane_off = static_cast<int64_t>(plane) * L * d;

    constexpr float LOG2E = 1.44269504088896340736f, LN2 = 0.69314718055994530942f;
    const float sc2 = p.scale * LOG2E;                // scores are kept in the base-2 domain
    // ---- this lane's slice of its query row, times scale * log2(e), as the B operand of the score MFMAs:
    // chunk c holds features 16 c + 8 half .. + 7 (zero past d / past L), split into three bf16 parts
    v8bf qb[NC][3];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int e0 = 16 * c + 8 * half;
        v4f x0 = {0.0f, 0.0f, 0.0f, 0.0f}, x1 = {0.0f, 0.0f, 0.0f, 0.0f};
        if (p.in_ld) {
            // [d][L]: one element per feature row, lanes along the queries (whole 128-byte runs)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (q < L && e0 + i < d) x0[i] = p.Q[plane_off + static_cast<int64_t>(e0 + i) * L + q];
                if (q < L && e0 + 4 + i < d) x1[i] = p.Q[plane_off + static_cast<int64_t>(e0 + 4 + i) * L + q];
            }
        } else {
            const float* qrow = p.Q + plane_off + static_cast<int64_t>(q) * d;
            if (q < L && e0 < d) x0 = *reinterpret_cast<const v4f*>(qrow + e0);
            if (q < L && e0 + 4 < d) x1 = *reinterpret_cast<const v4f*>(qrow + e0 + 4);
        }
        x0 *= sc2;
        x1 *= sc2;
        uint2 lo[3], hi[3];
        split4(x0, lo);
        split4(x1, hi);
#pragma unroll
        for (int part = 0; part < 3; ++part)
            qb[c][part] = __builtin_bit_cast(v8bf, v4i{static_cast<int>(lo[part].x), static_cast<int>(lo[part].y),
                                                      static_cast<int>(hi[part].x), static_cast<int>(hi[part].y)});
    }

    v16f acc_o[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc_o[b][r] = 0.0f;
    float m_run = -INFINITY, l_run = 0.0f;
    float m_head = -INFINITY;                          // maximum over the keys of the reference's first block
    const int row_keys = p.causal ? (q + 1 < L ? q + 1 : L) : L;     // keys this query may see
    const int head_keys = p.head < row_keys ? p.head : row_keys;
    // keys any query of this wave may see (wave-uniform)
    const int wave_keys = p.causal ? (q0 + 32 < L ? q0 + 32 : L) : L;
    // lanes past the last query read the last row (never stored)
    const float* bias_row = p.bias ? p.bias + (static_cast<int64_t>(plane) * L + (q < L ? q : L - 1)) * L : nullptr;

    // Bias of this lane's 16 keys of the tile starting at key0 (zeros past L), into bias_buf.  Rows of a
    // length that is no multiple of 4 are read with 16-byte loads all the same (4-byte aligned).
    float bias_buf[16];
    auto load_bias = [&](int key0) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int key = key0 + 8 * g + 4 * half;
            if (key + 3 < L) {
                const v4f x = *reinterpret_cast<const v4f_u*>(bias_row + key);
                bias_buf[4 * g] = x[0]; bias_buf[4 * g + 1] = x[1]; bias_buf[4 * g + 2] = x[2]; bias_buf[4 * g + 3] = x[3];
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) bias_buf[4 * g + i] = key + i < L ? bias_row[key + i] : 0.0f;
            }
        }
    };
    if (PF && bias_row && wave_active) load_bias(0);

    // One tile of 32 keys for the wave's 32 queries.  Scores live in the base-2 domain (the query slice
    // carries scale * log2(e)), so a probability is one subtraction and one v_exp_f32.
    auto do_tile = [&](auto plain_t, int kt, int key0) {
        constexpr bool PLAIN = decltype(plain_t)::value;
        // ---- bias of this lane's 16 keys, requested before the matrix work (or a tile ago)
        float bv[16];
        const bool has_bias = bias_row != nullptr;     // wave-uniform
        if (has_bias) {
            if (!PF) load_bias(key0);
#pragma unroll
            for (int r = 0; r < 16; ++r) bv[r] = bias_buf[r];
            if (PF && key0 + 32 < wave_keys) load_bias(key0 + 32);
        }
        // ---- S^T = K_tile . Q^T
        v16f st;
        const uint8_t* kfrag = lds_k + kt * KT_BYTES + lane * 16;     // each lane its 16 bytes of a fragment
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            v8bf ka[3];
#pragma unroll
            for (int part = 0; part < 3; ++part) ka[part] = *reinterpret_cast<const v8bf*>(kfrag + (c * 3 + part) * 1024);
#pragma unroll
            for (int t = 0; t < 6; ++t) {
                // the first product starts from the constant zero: no registers to clear
                const v16f zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                st = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[SPLIT_TERMS[t][0]], qb[c][SPLIT_TERMS[t][1]], (c == 0 && t == 0) ? zero : st, 0, 0, 0);
            }
        }
        // ---- scores of this lane's query: bias, masks; tile maximum
        float m_tile = -INFINITY;
        if (has_bias) {
#pragma unroll
            for (int r = 0; r < 16; ++r) st[r] = __builtin_fmaf(bv[r], LOG2E, st[r]);
        }
        if (!PLAIN) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int key = key0 + 8 * (r >> 2) + 4 * half + (r & 3);
                if (key >= row_keys) st[r] = -INFINITY;
                if (key < head_keys) m_head = fmaxf(m_head, st[r]);
            }
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) m_tile = fmaxf(m_tile, st[r]);
        m_tile = fmaxf(m_tile, lane_xor32(m_tile));
        const float m_new = fmaxf(m_run, m_tile);
        const float alpha = (m_run == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(m_run - m_new);
        const float m_sub = (m_new == -INFINITY) ? 0.0f : m_new;       // keeps -inf - -inf out of the exponent
        float l_tile = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            st[r] = __builtin_amdgcn_exp2f(st[r] - m_sub);
            l_tile += st[r];
        }
        l_tile += lane_xor32(l_tile);
        l_run = alpha * l_run + l_tile;
        m_run = m_new;
        // ---- O^T = alpha * O^T + V^T . P   (the rescale is skipped while no maximum of the wave moves)
        const bool rescale = __builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0;
        if (rescale) {
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc_o[b][r] *= alpha;
        }
        const uint8_t* vfrag = lds_v + kt * VT_BYTES + lane * 16;
#pragma unroll
        for (int ch = 0; ch < 2; ++ch) {
            // the probabilities of 16 keys as three bf16 parts: score registers 8 ch .. 8 ch + 7 of this lane
            uint2 lo[3], hi[3];
            split4(v4f{st[8 * ch], st[8 * ch + 1], st[8 * ch + 2], st[8 * ch + 3]}, lo);
            split4(v4f{st[8 * ch + 4], st[8 * ch + 5], st[8 * ch + 6], st[8 * ch + 7]}, hi);
            v8bf pb[3];
#pragma unroll
            for (int part = 0; part < 3; ++part)
                pb[part] = __builtin_bit_cast(v8bf, v4i{static_cast<int>(lo[part].x), static_cast<int>(lo[part].y),
                                                        static_cast<int>(hi[part].x), static_cast<int>(hi[part].y)});
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                v8bf va[3];
#pragma unroll
                for (int part = 0; part < 3; ++part) va[part] = *reinterpret_cast<const v8bf*>(vfrag + ((b * 2 + ch) * 3 + part) * 1024);
#pragma unroll
                for (int t = 0; t < 6; ++t)
                    acc_o[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[SPLIT_TERMS[t][0]], pb[SPLIT_TERMS[t][1]], acc_o[b], 0, 0, 0);
            }
        }
    };

    const int stage = p.stage_rows;
    for (int c0 = 0; c0 < L; c0 += stage) {
        // ---- stage keys c0 .. c0+stage-1 of K and V (zeros past L and past d; whole tiles of 32 only)
        __syncthreads();
        const int ckeys = L - c0 < stage ? L - c0 : stage;
        const int rows = (ckeys + 31) / 32 * 32;
        if (p.in_ld) {
            // source rows run along the keys: four keys of one feature per thread, scattered into the
            // key-major LDS tiles
            // (eight lanes read 128 contiguous bytes of one feature row; the LDS writes of a wave then
            // spread over 16 banks instead of 2)
            const int kq_n = rows / 4;
            for (int idx = tid; idx < DP * kq_n; idx += NW * 64) {
                const int rest = idx >> 3;
                const int dd = rest % DP, kq = ((rest / DP) * 8 + (idx & 7)) * 4;
                v4f kx = {0.0f, 0.0f, 0.0f, 0.0f}, vx = {0.0f, 0.0f, 0.0f, 0.0f};
                if (dd < d) {
                    const int64_t off = plane_off + static_cast<int64_t>(dd) * L + c0 + kq;
                    if (kq + 3 < ckeys) {
                        kx = *reinterpret_cast<const v4f_u*>(p.K + off);
                        vx = *reinterpret_cast<const v4f_u*>(p.V + off);
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            if (kq + i < ckeys) { kx[i] = p.K[off + i]; vx[i] = p.V[off + i]; }
                    }
                }
                // four keys of feature dd.  K: two bytes per key and part; V: the four keys are neighbours in
                // the lane slot of their feature (kq is a multiple of 4), eight bytes per part
                uint2 parts[3];
                split4(kx, parts);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int key = kq + i;
                    uint8_t* dst = lds_k + (key >> 5) * KT_BYTES + (dd >> 4) * 3072 + ((dd >> 3) & 1) * 512 + (key & 31) * 16 + (dd & 7) * 2;
#pragma unroll
                    for (int part = 0; part < 3; ++part) {
                        const uint32_t w = (i < 2 ? parts[part].x : parts[part].y) >> (16 * (i & 1));
                        *reinterpret_cast<uint16_t*>(dst + part * 1024) = static_cast<uint16_t>(w);
                    }
                }
                split4(vx, parts);
                {
                    const int kc = kq & 15;            // place of the first key in its chunk of 16
                    uint8_t* dst = lds_v + (kq >> 5) * VT_BYTES + (((dd >> 5) * 2 + ((kq >> 4) & 1)) * 3) * 1024 +
                                   (((kc >> 2) & 1) * 32 + (dd & 31)) * 16 + (kc >> 3) * 8;
#pragma unroll
                    for (int part = 0; part < 3; ++part) *reinterpret_cast<uint2*>(dst + part * 1024) = parts[part];
                }
            }
        } else {
            for (int idx = tid; idx < rows * (DP / 4); idx += NW * 64) {
                const int key = idx / (DP / 4), c = (idx % (DP / 4)) * 4;
                v4f kx = {0.0f, 0.0f, 0.0f, 0.0f}, vx = {0.0f, 0.0f, 0.0f, 0.0f};
                if (key < ckeys && c < d) {
                    const int64_t off = plane_off + static_cast<int64_t>(c0 + key) * d + c;
                    kx = *reinterpret_cast<const v4f*>(p.K + off);
                    vx = *reinterpret_cast<const v4f*>(p.V + off);
                }
                // features c .. c+3 of one key: eight bytes of each part's fragment
                uint2 parts[3];
                split4(kx, parts);
                uint8_t* dst = lds_k + (key >> 5) * KT_BYTES + (c >> 4) * 3072 + ((c >> 3) & 1) * 512 + (key & 31) * 16 + ((c >> 2) & 1) * 8;
#pragma unroll
                for (int part = 0; part < 3; ++part) *reinterpret_cast<uint2*>(dst + part * 1024) = parts[part];
                // V: features c .. c+3 of one key go to four lane slots of the fragments of V^T, two bytes each
                split4(vx, parts);
                {
                    const int kc = key & 15;
                    const int slot = 4 * (kc >> 3) + (kc & 3);
                    uint8_t* vdst = lds_v + (key >> 5) * VT_BYTES + (((c >> 5) * 2 + ((key >> 4) & 1)) * 3) * 1024 +
                                    (((kc >> 2) & 1) * 32 + (c & 31)) * 16 + slot * 2;
#pragma unroll
                    for (int i = 0; i < 4; ++i)
#pragma unroll
                        for (int part = 0; part < 3; ++part) {
                            const uint32_t w = (i < 2 ? parts[part].x : parts[part].y) >> (16 * (i & 1));
                            *reinterpret_cast<uint16_t*>(vdst + part * 1024 + i * 16) = static_cast<uint16_t>(w);
                        }
                }
            }
        }
        __syncthreads();
        if (!wave_active) continue;

        const int tiles_here = (ckeys + 31) / 32;
        for (int kt = 0; kt < tiles_here; ++kt) {
            const int key0 = c0 + kt * 32;             // first key of the tile
            if (key0 >= wave_keys) break;              // causal: nothing left for any query of the wave
            // A tile is plain when every query of the wave sees all 32 keys and the tile lies behind the
            // reference's first block; plain tiles skip the masks and the first-block bookkeeping.
            const bool plain = key0 + 32 <= L && (!p.causal || key0 + 32 <= q0 + 1) && key0 >= p.head;
            if (plain) do_tile(std::true_type{}, kt, key0);
            else do_tile(std::false_type{}, kt, key0);
        }
    }
    if (!wave_active || q >= L) return;

    // ---- finish the row.  The reference lets a first block of keys that is masked out entirely (all
    // of them -inf) poison the row: its sum becomes NaN and the row is written as O = 0, LSE = -inf
    // (FlashAttn.cpp:96-103, 121-131).  m_head reproduces that outcome.
    m_head = fmaxf(m_head, lane_xor32(m_head));
    const bool live = l_run > 0.0f && m_head > -INFINITY;
    const float inv = live ? 1.0f / (l_run + p.eps) : 0.0f;
    if (p.out_ld) {
        // [d][L]: lanes along the queries
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int dd = b * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                if (dd < d) p.O[plane_off + static_cast<int64_t>(dd) * L + q] = live ? acc_o[b][r] * inv : 0.0f;
            }
    } else {
        float* orow = p.O + plane_off + static_cast<int64_t>(q) * d;
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int dd = b * 32 + 8 * g + 4 * half;
                if (dd < d) {
                    const v4f o = {acc_o[b][4 * g] * inv, acc_o[b][4 * g + 1] * inv, acc_o[b][4 * g + 2] * inv, acc_o[b][4 * g + 3] * inv};
                    *reinterpret_cast<v4f*>(orow + dd) = live ? o : v4f{0.0f, 0.0f, 0.0f, 0.0f};
                }
            }
    }
    if (p.LSE && half == 0) p.LSE[static_cast<int64_t>(plane) * L + q] = live ? m_run * LN2 + __logf(l_run + p.eps) : -INFINITY;
}

template <int DP, int NW, bool PF>
int launch_flash(AttnParams p, hipStream_t stream) {
    using T = AttnTiling<DP, NW>;
    auto kernel = &flash_attn_forward_kernel<DP, NW, PF>;
    const int l32 = (p.L + 31) / 32 * 32;
    p.stage_rows = l32 < T::CH ? l32 : T::CH;
    const size_t lds = static_cast<size_t>(p.stage_rows / 32) * (T::KT_BYTES + T::VT_BYTES);
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(T::lds_bytes));
    if (attr != hipSuccess) {
        (void)hipGetLastError();
        set_error("flash_attn_forward_hip: cannot reserve %zu bytes of LDS", T::lds_bytes);
        return RC_LAUNCH;
    }
    const dim3 grid((p.L + 32 * NW - 1) / (32 * NW), p.planes), block(NW * 64);
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, p);
    return check_launch("flash_attn_forward_kernel");
}

}  // namespace
}  // namespace ppmlhip

using namespace ppmlhip;

extern "C" int flash_attn_forward_ex_hip(int B, int h, int L, int d, int causal, float scale, float softmax_eps, int Bc,
                                         const float* Q, const float* K, const float* V, const float* bias,
                                         float* O, float* LSE, int layout, ppml_hip_stream_t stream) {
    if (!Q || !K || !V || !O || B <= 0 || h <= 0 || L <= 0 || d <= 0) {
        set_error("flash_attn_forward_hip: bad arguments (B=%d h=%d L=%d d=%d)", B, h, L, d);
        return RC_BAD_ARGS;
    }
    if (d > 64 || (d & 3) != 0) {                     // the rule of src/backend/CUDABackend.cpp:457-463
        set_error("flash_attn_forward_hip: head dimension %d not supported (multiple of 4, at most 64)", d);
        return RC_BAD_ARGS;
    }
    const auto misaligned = [](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) != 0; };
    if (layout < 0 || layout > 3) { set_error("flash_attn_forward_hip: layout %d is not 0..3", layout); return RC_BAD_ARGS; }
    if (misaligned(Q) || misaligned(K) || misaligned(V) || misaligned(O)) {
        set_error("flash_attn_forward_hip: Q, K, V and O must be 16-byte aligned");
        return RC_BAD_ARGS;
    }
    const int64_t planes = static_cast<int64_t>(B) * h;
    if (planes > 65535) {
        set_error("flash_attn_forward_hip: %lld planes exceed the grid limit of 65535", static_cast<long long>(planes));
        return RC_BAD_ARGS;
    }
    AttnParams p;
    p.Q = Q; p.K = K; p.V = V; p.bias = bias; p.O = O; p.LSE = LSE;
    p.planes = static_cast<int>(planes); p.L = L; p.d = d;
    p.causal = causal ? 1 : 0;
    p.scale = scale > 0.0f ? scale : 1.0f / std::sqrt(static_cast<float>(d));   // FlashAttn.cpp:63
    p.eps = softmax_eps;
    p.head = Bc > 0 ? Bc : 64;                        // FlashAttn.cpp:62
    p.stage_rows = 0;                                 // set per instance
    p.in_ld = layout & 1;
    p.out_ld = (layout >> 1) & 1;
    StatsScope stat("hip/flash_attn", static_cast<int64_t>(planes) * L, d, L, static_cast<hipStream_t>(stream));
    hipStream_t s = static_cast<hipStream_t>(stream);
    // Four-wave work-groups (128 queries): 824 planes of 256 queries make 1648 of them, which spread over
    // 256 CUs more evenly than 824 eight-wave ones (6.4 per CU against 3.2, each rounded up).
    const bool short_rows = L <= 128;
    if (d <= 32) return short_rows ? launch_flash<32, 4, true>(p, s) : launch_flash<32, 4, false>(p, s);
    return short_rows ? launch_flash<64, 4, true>(p, s) : launch_flash<64, 4, false>(p, s);
}

extern "C" int flash_attn_forward_hip(int B, int h, int L, int d, int causal, float scale, float softmax_eps, int Bc,
                                      const float* Q, const float* K, const float* V, const float* bias,
                                      float* O, float* LSE, ppml_hip_stream_t stream) {
    return flash_attn_forward_ex_hip(B, h, L, d, causal, scale, softmax_eps, Bc, Q, K, V, bias, O, LSE, 0, stream);
}
