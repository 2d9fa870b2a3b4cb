// Fused attention backward for gfx950: the twin of the reference's flash_attn_backward_cuda
// (include/ppml/FlashAttn.h:97-101, declared src/backend/CUDAKernels.cpp:176-179, called from
// kernel_flash_attn_back_cuda, 905-924) with the mathematics of flash_attn_backward_cpu
// (src/ops/FlashAttn.cpp:140-210):
//     P = exp(S - LSE)          S = scale * Q K^T + bias           D_i = sum_d dO_id O_id
//     dS = P * (dO V^T - D)     dQ = scale * dS K     dK = scale * dS^T Q     dV = P^T dO     dbias = dS
// Nothing is stored between forward and backward but O and LSE; P is recomputed per 32 x 32 tile.
//
// Two kernels, each the forward kernel's arrangement (see attention.hip) with one side held in registers:
//   * rows kernel  (dQ, dbias): a wave owns 32 queries; scores and dO V^T are computed transposed, so a lane
//     holds 16 keys of ITS query: D_i and LSE_i are per-lane scalars, dS is ready as the B operand of
//     dQ^T += K^T dS, and dbias is written from the registers;
//   * columns kernel (dK, dV): a wave owns 32 keys; scores and dO V^T are computed un-transposed, so a lane
//     holds 16 queries of ITS key: P and dS are ready as the B operands of dV^T += dO^T P and
//     dK^T += Q^T dS; LSE and D of the tile's queries come from LDS.
// All five contractions run on the bf16 matrix pipe at binary32 accuracy (exact three-way split of every
// operand, six partial products per 16 contracted elements; common.hpp): the streamed side lies in LDS as ready
// MFMA fragments, in two arrangements where it is contracted both ways (over the features for S and dO V^T,
// over its rows for the gradients), the held side and the freshly computed P / dS are split in registers.
// No atomics and no scratch memory: every output element has one owner, so the results do not depend on
// scheduling (the reference's CUDA path accumulates dK and dV with atomicAdd).
#include "common.hpp"

#include <cmath>
#include <type_traits>

namespace ppmlhip {
namespace {

constexpr float LOG2E = 1.44269504088896340736f;

struct AttnBackParams {
    const float* Q; const float* K; const float* V; const float* bias;
    const float* O; const float* dO; const float* LSE;
    float* dQ; float* dK; float* dV; float* dbias;
    int planes, L, d;
    int causal;
    float scale;
    int stage_rows;      // rows of the streamed side staged in LDS at a time (a multiple of 32)
};

__device__ __forceinline__ float lane_xor32(float x) { return __shfl_xor(x, 32, 64); }

template <int DP> struct BackTiling {
    static constexpr int NC = DP / 16;                // 16-feature chunks of a contraction over the features
    static constexpr int NB = DP / 32;                // 32-feature blocks of a transposed gradient
    // A 32-row tile of a streamed matrix in LDS, as 1 KB MFMA operand fragments (lane l reads bytes 16 l ..):
    //   "row" fragments, one per (chunk, part): lane (row, half) holds features 16 c + 8 half .. + 7 of its row;
    //   "column" fragments of the transpose, one per (feature block, 16-row chunk, part): slot i of lane
    //   (feature, half) holds row 16 ch + 8 (i / 4) + 4 half + i % 4 -- the order in which the accumulator
    //   registers 8 ch .. 8 ch + 7 of a 32 x 32 product hold the rows.
    static constexpr int ROW_BYTES = NC * 3 * 1024;
    static constexpr int COL_BYTES = NB * 2 * 3 * 1024;
    static constexpr int CH_ROWS = 64;                // rows staged at a time by the rows kernel (K both ways, V by rows)
    static constexpr int CH_COLS = 96;                // ... by the columns kernel (Q and dO both ways)
};

__device__ __forceinline__ v8bf pack_parts(const uint2& lo, const uint2& hi) {
    return __builtin_bit_cast(v8bf, v4i{static_cast<int>(lo.x), static_cast<int>(lo.y), static_cast<int>(hi.x), static_cast<int>(hi.y)});
}

// This lane's slice of row `row` of a [L][d] matrix times `factor`, as the B operand of a contraction over the
// features: chunk c holds features 16 c + 8 half .. + 7 (zero past d and past L), split into three bf16 parts.
template <int DP>
__device__ __forceinline__ void load_slice_parts(const float* base, int row, int L, int d, int half, float factor,
                                                 v8bf (&out)[DP / 16][3]) {
#pragma unroll
    for (int c = 0; c < DP / 16; ++c) {
        const int e0 = 16 * c + 8 * half;
        v4f x0 = {0.0f, 0.0f, 0.0f, 0.0f}, x1 = {0.0f, 0.0f, 0.0f, 0.0f};
        const float* src = base + static_cast<int64_t>(row) * d;
        if (row < L && e0 < d) x0 = *reinterpret_cast<const v4f*>(src + e0);
        if (row < L && e0 + 4 < d) x1 = *reinterpret_cast<const v4f*>(src + e0 + 4);
        x0 *= factor;
        x1 *= factor;
        uint2 lo[3], hi[3];
        split4(x0, lo);
        split4(x1, hi);
#pragma unroll
        for (int part = 0; part < 3; ++part) out[c][part] = pack_parts(lo[part], hi[part]);
    }
}

// Writes features c .. c+3 of row `row` of a staged matrix into its fragments: row fragments at lds_row and / or
// column fragments at lds_col (null = not wanted).
template <int DP>
__device__ __forceinline__ void put_fragments(const v4f& x, int row, int c, uint8_t* lds_row, uint8_t* lds_col) {
    using T = BackTiling<DP>;
    uint2 parts[3];
    split4(x, parts);
    if (lds_row) {
        // eight bytes of each part's fragment
        uint8_t* dst = lds_row + (row >> 5) * T::ROW_BYTES + (c >> 4) * 3072 + ((c >> 3) & 1) * 512 + (row & 31) * 16 + ((c >> 2) & 1) * 8;
#pragma unroll
        for (int part = 0; part < 3; ++part) *reinterpret_cast<uint2*>(dst + part * 1024) = parts[part];
    }
    if (lds_col) {
        // the same four features go to four lane slots of the transposed fragments, two bytes each
        const int kc = row & 15;
        const int slot = 4 * (kc >> 3) + (kc & 3);
        uint8_t* dst = lds_col + (row >> 5) * T::COL_BYTES + (((c >> 5) * 2 + ((row >> 4) & 1)) * 3) * 1024 +
                       (((kc >> 2) & 1) * 32 + (c & 31)) * 16 + slot * 2;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int part = 0; part < 3; ++part) {
                const uint32_t w = (i < 2 ? parts[part].x : parts[part].y) >> (16 * (i & 1));
                *reinterpret_cast<uint16_t*>(dst + part * 1024 + i * 16) = static_cast<uint16_t>(w);
            }
    }
}

// Stages rows r0 .. r0+rows-1 (at most MAXROWS) of two [L][d] matrices into LDS as fragments (zeros past `valid`
// rows and past d).  Every load of the stage is issued before the first value is used: a work-group waits for
// one memory round trip per stage, not one per loop iteration.
template <int DP, int NT, int MAXROWS>
__device__ __forceinline__ void stage_two(const float* a, uint8_t* a_row, uint8_t* a_col,
                                          const float* b, uint8_t* b_row, uint8_t* b_col,
                                          int r0, int rows, int valid, int d, int tid) {
    constexpr int NI = (MAXROWS * (DP / 4) + NT - 1) / NT;
    v4f xa[NI], xb[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int idx = tid + i * NT;
        const int row = idx / (DP / 4), c = (idx % (DP / 4)) * 4;
        xa[i] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
        xb[i] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
        if (row < valid && c < d) {
            const int64_t off = static_cast<int64_t>(r0 + row) * d + c;
            xa[i] = *reinterpret_cast<const v4f*>(a + off);
            xb[i] = *reinterpret_cast<const v4f*>(b + off);
        }
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int idx = tid + i * NT;
        const int row = idx / (DP / 4), c = (idx % (DP / 4)) * 4;
        if (row < rows) {
            put_fragments<DP>(xa[i], row, c, a_row, a_col);
            put_fragments<DP>(xb[i], row, c, b_row, b_col);
        }
    }
}

// acc(32 x 32) = tile(32 rows x DP, row fragments in LDS, rows = accumulator rows) . slice^T (this lane's column);
// `frags` points at this lane's 16 bytes of the tile's first fragment
template <int DP>
__device__ __forceinline__ v16f tile_times_slice(const uint8_t* frags, const v8bf (&slice)[DP / 16][3]) {
    v16f acc;
#pragma unroll
    for (int c = 0; c < DP / 16; ++c) {
        v8bf a[3];
#pragma unroll
        for (int part = 0; part < 3; ++part) a[part] = *reinterpret_cast<const v8bf*>(frags + (c * 3 + part) * 1024);
#pragma unroll
        for (int t = 0; t < 6; ++t) {
            // the first product starts from the constant zero: no registers to clear
            const v16f zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[SPLIT_TERMS[t][0]], slice[c][SPLIT_TERMS[t][1]], (c == 0 && t == 0) ? zero : acc, 0, 0, 0);
        }
    }
    return acc;
}

// out^T(DP features x 32 columns) += tile^T . w, contracting the 32 rows of the tile in the order in which the
// accumulator registers of `w` hold them; `frags` points at this lane's 16 bytes of the tile's first column fragment.
template <int DP>
__device__ __forceinline__ void accumulate_transposed(v16f (&out)[DP / 32], const uint8_t* frags, const v16f& w) {
#pragma unroll
    for (int ch = 0; ch < 2; ++ch) {
        uint2 lo[3], hi[3];
        split4(v4f{w[8 * ch], w[8 * ch + 1], w[8 * ch + 2], w[8 * ch + 3]}, lo);
        split4(v4f{w[8 * ch + 4], w[8 * ch + 5], w[8 * ch + 6], w[8 * ch + 7]}, hi);
        v8bf wb[3];
#pragma unroll
        for (int part = 0; part < 3; ++part) wb[part] = pack_parts(lo[part], hi[part]);
#pragma unroll
        for (int b = 0; b < DP / 32; ++b) {
            v8bf a[3];
#pragma unroll
            for (int part = 0; part < 3; ++part) a[part] = *reinterpret_cast<const v8bf*>(frags + ((b * 2 + ch) * 3 + part) * 1024);
#pragma unroll
            for (int t = 0; t < 6; ++t)
                out[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[SPLIT_TERMS[t][0]], wb[SPLIT_TERMS[t][1]], out[b], 0, 0, 0);
        }
    }
}

// ------------------------------------------------------------------------------------------------------------
// dQ and dbias: a wave owns 32 queries and walks over the keys.
template <int DP, int NW>
__global__ __launch_bounds__(NW * 64) void flash_attn_back_rows_kernel(const AttnBackParams p) {
    using T = BackTiling<DP>;
    constexpr int NB = T::NB, NC = T::NC;
    extern __shared__ __attribute__((aligned(16))) uint8_t back_lds[];
    const int tiles_staged = p.stage_rows / 32;
    uint8_t* lds_k_row = back_lds;                                  // K by rows: S^T = K . Q^T
    uint8_t* lds_k_col = lds_k_row + tiles_staged * T::ROW_BYTES;   // K^T: dQ^T += K^T . dS
    uint8_t* lds_v_row = lds_k_col + tiles_staged * T::COL_BYTES;   // V by rows: (dO V^T)^T = V . dO^T
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 31, half = lane >> 5;
    const int plane = blockIdx.y, L = p.L, d = p.d;
    const int q0 = (blockIdx.x * NW + wave) * 32, q = q0 + j;
    const bool wave_active = q0 < L;
    const int64_t po = static_cast<int64_t>(plane) * L * d;

    v8bf qb[NC][3], dob[NC][3];
    load_slice_parts<DP>(p.Q + po, q, L, d, half, p.scale * LOG2E, qb);
    load_slice_parts<DP>(p.dO + po, q, L, d, half, 1.0f, dob);
    // D_i = sum_d dO_id * O_id: this lane's half of the features, then the other half from lane j + 32
    float D_i = 0.0f;
    if (q < L) {
#pragma unroll
        for (int c = 0; c < NC; ++c)
#pragma unroll
            for (int e = 16 * c + 8 * half; e < 16 * c + 8 * half + 8; e += 4) {
                if (e >= d) continue;
                const v4f a = *reinterpret_cast<const v4f*>(p.dO + po + static_cast<int64_t>(q) * d + e);
                const v4f o = *reinterpret_cast<const v4f*>(p.O + po + static_cast<int64_t>(q) * d + e);
                D_i += a[0] * o[0] + a[1] * o[1] + a[2] * o[2] + a[3] * o[3];
            }
    }
    D_i += lane_xor32(D_i);
    const float lse = q < L ? p.LSE[static_cast<int64_t>(plane) * L + q] : -INFINITY;
    // a row without any visible key (LSE = -inf) has no gradient: +inf makes every probability exp2(-inf) = 0
    const float lse2 = lse > -INFINITY ? lse * LOG2E : INFINITY;
    const int row_keys = p.causal ? (q + 1 < L ? q + 1 : L) : L;
    const int wave_keys = p.causal ? (q0 + 32 < L ? q0 + 32 : L) : L;
    const float* bias_row = p.bias ? p.bias + (static_cast<int64_t>(plane) * L + (q < L ? q : L - 1)) * L : nullptr;
    float* dbias_row = p.dbias ? p.dbias + (static_cast<int64_t>(plane) * L + (q < L ? q : L - 1)) * L : nullptr;

    v16f acc_q[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc_q[b][r] = 0.0f;

    // Bias of this lane's 16 keys of the tile that starts at key0 (zeros past L), 16 bytes at a time.
    float bv[16];
    const auto load_bias = [&](int key0) {
        if (!bias_row) return;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int key = key0 + 8 * g + 4 * half;
            if (key + 3 < L) {
                const v4f x = *reinterpret_cast<const v4f_u*>(bias_row + key);
                bv[4 * g] = x[0]; bv[4 * g + 1] = x[1]; bv[4 * g + 2] = x[2]; bv[4 * g + 3] = x[3];
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) bv[4 * g + i] = key + i < L ? bias_row[key + i] : 0.0f;
            }
        }
    };
    if (wave_active) load_bias(0);

    const int stage = p.stage_rows;
    for (int c0 = 0; c0 < L; c0 += stage) {
        __syncthreads();
        const int ckeys = L - c0 < stage ? L - c0 : stage;
        const int rows = (ckeys + 31) / 32 * 32;
        stage_two<DP, NW * 64, T::CH_ROWS>(p.K + po, lds_k_row, lds_k_col, p.V + po, lds_v_row, nullptr, c0, rows, ckeys, d, tid);
        __syncthreads();
        if (!wave_active) continue;
        for (int kt = 0; kt < rows / 32; ++kt) {
            const int key0 = c0 + kt * 32;
            // ---- probabilities of this lane's query for its 16 keys of the tile (their bias was requested a
            // tile ago, see below)
            v16f st = tile_times_slice<DP>(lds_k_row + kt * T::ROW_BYTES + lane * 16, qb);
            v16f dp = tile_times_slice<DP>(lds_v_row + kt * T::ROW_BYTES + lane * 16, dob);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int key = key0 + 8 * (r >> 2) + 4 * half + (r & 3);
                float s2 = st[r];
                if (bias_row) s2 = __builtin_fmaf(bv[r], LOG2E, s2);
                const float pr = key < row_keys ? __builtin_amdgcn_exp2f(s2 - lse2) : 0.0f;
                st[r] = pr * (dp[r] - D_i);            // dS
            }
            // the bias registers are free again: the next tile's values travel during the rest of this tile
            // and the first contractions of the next (the tiles follow each other across the stages)
            if (key0 + 32 < L) load_bias(key0 + 32);
            // ---- dbias = dS (zeros where the key is masked; every position of a valid row is written)
            if (dbias_row && q < L) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int key = key0 + 8 * g + 4 * half;
                    if (key + 3 < L) {
                        *reinterpret_cast<v4f_u*>(dbias_row + key) = v4f{st[4 * g], st[4 * g + 1], st[4 * g + 2], st[4 * g + 3]};
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; ++i) if (key + i < L) dbias_row[key + i] = st[4 * g + i];
                    }
                }
            }
            if (key0 >= wave_keys) continue;           // causal: no query of the wave sees this tile (dS = 0)
            // ---- dQ^T += K^T . dS
            if (p.dQ) accumulate_transposed<DP>(acc_q, lds_k_col + kt * T::COL_BYTES + lane * 16, st);
        }
    }
    if (!wave_active || q >= L || !p.dQ) return;
    float* row = p.dQ + po + static_cast<int64_t>(q) * d;
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int dd = b * 32 + 8 * g + 4 * half;
            if (dd < d)
                *reinterpret_cast<v4f*>(row + dd) = v4f{acc_q[b][4 * g] * p.scale, acc_q[b][4 * g + 1] * p.scale,
                                                        acc_q[b][4 * g + 2] * p.scale, acc_q[b][4 * g + 3] * p.scale};
        }
}

// ------------------------------------------------------------------------------------------------------------
// dK and dV: a wave owns 32 keys and walks over the queries.
template <int DP, int NW>
__global__ __launch_bounds__(NW * 64) void flash_attn_back_cols_kernel(const AttnBackParams p) {
    using T = BackTiling<DP>;
    constexpr int NB = T::NB, NC = T::NC;
    extern __shared__ __attribute__((aligned(16))) uint8_t back_lds[];
    const int tiles_staged = p.stage_rows / 32;
    uint8_t* lds_q_row = back_lds;                                   // Q by rows: S = Q . K^T
    uint8_t* lds_q_col = lds_q_row + tiles_staged * T::ROW_BYTES;    // Q^T: dK^T += Q^T . dS
    uint8_t* lds_do_row = lds_q_col + tiles_staged * T::COL_BYTES;   // dO by rows: dO . V^T
    uint8_t* lds_do_col = lds_do_row + tiles_staged * T::ROW_BYTES;  // dO^T: dV^T += dO^T . P
    float* lds_lse = reinterpret_cast<float*>(lds_do_col + tiles_staged * T::COL_BYTES);   // LSE * log2(e) of the staged queries (+inf for dead rows)
    float* lds_D = lds_lse + p.stage_rows;             // D of the staged queries
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 31, half = lane >> 5;
    const int plane = blockIdx.y, L = p.L, d = p.d;
    const int k0w = (blockIdx.x * NW + wave) * 32, key = k0w + j;       // this lane's key
    const bool wave_active = k0w < L;
    const int64_t po = static_cast<int64_t>(plane) * L * d;

    v8bf kb[NC][3], vb[NC][3];
    load_slice_parts<DP>(p.K + po, key, L, d, half, p.scale * LOG2E, kb);
    load_slice_parts<DP>(p.V + po, key, L, d, half, 1.0f, vb);
    const float* bias_plane = p.bias ? p.bias + static_cast<int64_t>(plane) * L * L : nullptr;

    v16f acc_k[NB], acc_v[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) { acc_k[b][r] = 0.0f; acc_v[b][r] = 0.0f; }

    const int stage = p.stage_rows;
    // causal: queries before the wave's first key see none of its keys
    const int first_chunk = p.causal ? (k0w / stage) * stage : 0;
    for (int c0 = 0; c0 < L; c0 += stage) {
        __syncthreads();
        const int cq = L - c0 < stage ? L - c0 : stage;
        const int rows = (cq + 31) / 32 * 32;
        // Q and dO as fragments, and LSE and D = sum_d dO * O of the staged queries, from one batch of loads: a
        // thread holds four features of a row, the eight threads of a row add up their parts of D.
        {
            constexpr int NT = NW * 64, NI = (T::CH_COLS * (DP / 4) + NT - 1) / NT;
            static_assert(DP / 4 == 8 || DP / 4 == 16, "eight or sixteen threads per staged row");
            v4f xq[NI], xdo[NI], xo[NI];
            float lse_in[NI];
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                const int idx = tid + i * NT;
                const int row = idx / (DP / 4), c = (idx % (DP / 4)) * 4;
                xq[i] = xdo[i] = xo[i] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
                lse_in[i] = -INFINITY;
                if (row < cq) {
                    if (c < d) {
                        const int64_t off = po + static_cast<int64_t>(c0 + row) * d + c;
                        xq[i] = *reinterpret_cast<const v4f*>(p.Q + off);
                        xdo[i] = *reinterpret_cast<const v4f*>(p.dO + off);
                        xo[i] = *reinterpret_cast<const v4f*>(p.O + off);
                    }
                    if (c == 0) lse_in[i] = p.LSE[static_cast<int64_t>(plane) * L + c0 + row];
                }
            }
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                const int idx = tid + i * NT;
                const int row = idx / (DP / 4), c = (idx % (DP / 4)) * 4;
                float sum = xdo[i][0] * xo[i][0] + xdo[i][1] * xo[i][1] + xdo[i][2] * xo[i][2] + xdo[i][3] * xo[i][3];
                sum += __shfl_xor(sum, 1, 64);
                sum += __shfl_xor(sum, 2, 64);
                sum += __shfl_xor(sum, 4, 64);
                if (DP / 4 == 16) sum += __shfl_xor(sum, 8, 64);
                if (row < rows) {
                    put_fragments<DP>(xq[i], row, c, lds_q_row, lds_q_col);
                    put_fragments<DP>(xdo[i], row, c, lds_do_row, lds_do_col);
                    if (c == 0) {
                        lds_lse[row] = lse_in[i] > -INFINITY ? lse_in[i] * LOG2E : INFINITY;
                        lds_D[row] = sum;
                    }
                }
            }
        }
        __syncthreads();
        if (!wave_active || c0 < first_chunk) continue;
        for (int qt = 0; qt < rows / 32; ++qt) {
            const int qbase = c0 + qt * 32;
            if (p.causal && qbase + 32 <= k0w) continue;           // every query of the tile precedes every key of the wave
            // bias of this lane's key for its 16 queries of the tile, requested before the matrix work
            float bv[16];
            if (bias_plane) {
                const float* bcol = bias_plane + (key < L ? key : L - 1);
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int qq = qbase + 8 * (r >> 2) + 4 * half + (r & 3);
                    bv[r] = bcol[static_cast<int64_t>(qq < L ? qq : L - 1) * L];
                }
            }
            // ---- S[query][key] and dO V^T, un-transposed: this lane's key, 16 of the tile's queries
            v16f st = tile_times_slice<DP>(lds_q_row + qt * T::ROW_BYTES + lane * 16, kb);
            v16f dp = tile_times_slice<DP>(lds_do_row + qt * T::ROW_BYTES + lane * 16, vb);
            v16f ds;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const v4f lse4 = *reinterpret_cast<const v4f*>(lds_lse + qt * 32 + 8 * g + 4 * half);
                const v4f D4 = *reinterpret_cast<const v4f*>(lds_D + qt * 32 + 8 * g + 4 * half);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int r = 4 * g + i;
                    const int qq = qbase + 8 * g + 4 * half + i;
                    float s2 = st[r];
                    if (bias_plane) s2 = __builtin_fmaf(bv[r], LOG2E, s2);
                    const bool seen = qq < L && (!p.causal || key <= qq);
                    const float pr = seen ? __builtin_amdgcn_exp2f(s2 - lse4[i]) : 0.0f;
                    st[r] = pr;                                    // P
                    ds[r] = pr * (dp[r] - D4[i]);                  // dS
                }
            }
            // ---- dV^T += dO^T . P,  dK^T += Q^T . dS
            if (p.dV) accumulate_transposed<DP>(acc_v, lds_do_col + qt * T::COL_BYTES + lane * 16, st);
            if (p.dK) accumulate_transposed<DP>(acc_k, lds_q_col + qt * T::COL_BYTES + lane * 16, ds);
        }
    }
    if (!wave_active || key >= L) return;
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int dd = b * 32 + 8 * g + 4 * half;
            if (dd >= d) continue;
            const int64_t off = po + static_cast<int64_t>(key) * d + dd;
            if (p.dK) *reinterpret_cast<v4f*>(p.dK + off) = v4f{acc_k[b][4 * g] * p.scale, acc_k[b][4 * g + 1] * p.scale,
                                                                acc_k[b][4 * g + 2] * p.scale, acc_k[b][4 * g + 3] * p.scale};
            if (p.dV) *reinterpret_cast<v4f*>(p.dV + off) = v4f{acc_v[b][4 * g], acc_v[b][4 * g + 1], acc_v[b][4 * g + 2], acc_v[b][4 * g + 3]};
        }
}

template <int DP>
int launch_back(AttnBackParams p, hipStream_t stream) {
    using T = BackTiling<DP>;
    constexpr int NW = 4;
    const int l32 = (p.L + 31) / 32 * 32;
    const dim3 grid((p.L + 32 * NW - 1) / (32 * NW), p.planes), block(NW * 64);
    if (p.dQ || p.dbias) {
        p.stage_rows = l32 < T::CH_ROWS ? l32 : T::CH_ROWS;
        const size_t lds = static_cast<size_t>(p.stage_rows / 32) * (2 * T::ROW_BYTES + T::COL_BYTES);
        static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&flash_attn_back_rows_kernel<DP, NW>),
                                                           hipFuncAttributeMaxDynamicSharedMemorySize,
                                                           (T::CH_ROWS / 32) * (2 * T::ROW_BYTES + T::COL_BYTES));
        if (attr != hipSuccess) {
            (void)hipGetLastError();
            set_error("flash_attn_backward_hip: cannot reserve the LDS of the rows kernel");
            return RC_LAUNCH;
        }
        hipLaunchKernelGGL((flash_attn_back_rows_kernel<DP, NW>), grid, block, lds, stream, p);
        const int rc = check_launch("flash_attn_back_rows_kernel");
        if (rc != RC_OK) return rc;
    }
    if (p.dK || p.dV) {
        p.stage_rows = l32 < T::CH_COLS ? l32 : T::CH_COLS;
        const size_t lds = static_cast<size_t>(p.stage_rows / 32) * (2 * T::ROW_BYTES + 2 * T::COL_BYTES) +
                           static_cast<size_t>(p.stage_rows) * 2 * sizeof(float);
        static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&flash_attn_back_cols_kernel<DP, NW>),
                                                           hipFuncAttributeMaxDynamicSharedMemorySize,
                                                           (T::CH_COLS / 32) * (2 * T::ROW_BYTES + 2 * T::COL_BYTES) + T::CH_COLS * 8);
        if (attr != hipSuccess) {
            (void)hipGetLastError();
            set_error("flash_attn_backward_hip: cannot reserve the LDS of the columns kernel");
            return RC_LAUNCH;
        }
        hipLaunchKernelGGL((flash_attn_back_cols_kernel<DP, NW>), grid, block, lds, stream, p);
        return check_launch("flash_attn_back_cols_kernel");
    }
    return RC_OK;
}

}  // namespace
}  // namespace ppmlhip

using namespace ppmlhip;

extern "C" int flash_attn_backward_hip(int B, int h, int L, int d, int causal, float scale,
                                       const float* Q, const float* K, const float* V, const float* bias,
                                       const float* O, const float* dO, const float* LSE,
                                       float* dQ, float* dK, float* dV, float* dbias, ppml_hip_stream_t stream) {
    if (!Q || !K || !V || !O || !dO || !LSE || (!dQ && !dK && !dV && !dbias) || B <= 0 || h <= 0 || L <= 0 || d <= 0) {
        set_error("flash_attn_backward_hip: bad arguments (B=%d h=%d L=%d d=%d)", B, h, L, d);
        return RC_BAD_ARGS;
    }
    if (d > 64 || (d & 3) != 0) {
        set_error("flash_attn_backward_hip: head dimension %d not supported (multiple of 4, at most 64)", d);
        return RC_BAD_ARGS;
    }
    const auto misaligned = [](const void* ptr) { return ptr && (reinterpret_cast<uintptr_t>(ptr) & 15) != 0; };
    if (misaligned(Q) || misaligned(K) || misaligned(V) || misaligned(O) || misaligned(dO) || misaligned(dQ) || misaligned(dK) || misaligned(dV)) {
        set_error("flash_attn_backward_hip: Q, K, V, O, dO and the gradients must be 16-byte aligned");
        return RC_BAD_ARGS;
    }
    const int64_t planes = static_cast<int64_t>(B) * h;
    if (planes > 65535) {
        set_error("flash_attn_backward_hip: %lld planes exceed the grid limit of 65535", static_cast<long long>(planes));
        return RC_BAD_ARGS;
    }
    AttnBackParams p;
    p.Q = Q; p.K = K; p.V = V; p.bias = bias; p.O = O; p.dO = dO; p.LSE = LSE;
    p.dQ = dQ; p.dK = dK; p.dV = dV; p.dbias = dbias;
    p.planes = static_cast<int>(planes); p.L = L; p.d = d;
    p.causal = causal ? 1 : 0;
    p.scale = scale > 0.0f ? scale : 1.0f / std::sqrt(static_cast<float>(d));   // FlashAttn.cpp:153
    p.stage_rows = 0;
    StatsScope stat("hip/flash_attn_back", static_cast<int64_t>(planes) * L, d, L, static_cast<hipStream_t>(stream));
    hipStream_t s = static_cast<hipStream_t>(stream);
    return d <= 32 ? launch_back<32>(p, s) : launch_back<64>(p, s);
}
