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
    static constexpr int KS = DP + 4;                 // row pitch of the LDS tiles (floats): 16-byte reads, rows 4 banks apart
    static constexpr int CH = DP <= 32 ? 128 : 64;    // rows staged at a time
};

// This lane's slice of row `row` of a [L][d] matrix: elements half*DP/2 + s, zero past d and past L.
template <int DP>
__device__ __forceinline__ void load_slice(const float* base, int row, int L, int d, int half, float factor, float (&reg)[DP / 2]) {
#pragma unroll
    for (int s = 0; s < DP / 2; s += 4) {
        const int e = half * (DP / 2) + s;
        v4f x = {0.0f, 0.0f, 0.0f, 0.0f};
        if (row < L && e < d) x = *reinterpret_cast<const v4f*>(base + static_cast<int64_t>(row) * d + e);
        reg[s] = x[0] * factor; reg[s + 1] = x[1] * factor; reg[s + 2] = x[2] * factor; reg[s + 3] = x[3] * factor;
    }
}

// Stages rows r0 .. r0+rows-1 of two [L][d] matrices into LDS tiles of pitch KS (zeros past L and past d).
template <int DP, int NT>
__device__ __forceinline__ void stage_pair(const float* a, const float* b, float* lds_a, float* lds_b,
                                           int r0, int rows, int valid, int d, int tid) {
    constexpr int KS = BackTiling<DP>::KS;
    for (int idx = tid; idx < rows * (DP / 4); idx += NT) {
        const int row = idx / (DP / 4), c = (idx % (DP / 4)) * 4;
        v4f ax = {0.0f, 0.0f, 0.0f, 0.0f}, bx = {0.0f, 0.0f, 0.0f, 0.0f};
        if (row < valid && c < d) {
            const int64_t off = static_cast<int64_t>(r0 + row) * d + c;
            ax = *reinterpret_cast<const v4f*>(a + off);
            bx = *reinterpret_cast<const v4f*>(b + off);
        }
        *reinterpret_cast<v4f*>(lds_a + row * KS + c) = ax;
        *reinterpret_cast<v4f*>(lds_b + row * KS + c) = bx;
    }
}

// acc(32 x 32) = tile(32 rows x DP, from LDS, rows = accumulator rows) . slice^T (this lane's column)
template <int DP>
__device__ __forceinline__ v16f tile_times_slice(const float* tile_row, const float (&slice)[DP / 2]) {
    v16f acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
#pragma unroll
    for (int s = 0; s < DP / 2; s += 4) {
        const v4f x = *reinterpret_cast<const v4f*>(tile_row + s);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x[0], slice[s], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x[1], slice[s + 1], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x[2], slice[s + 2], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x[3], slice[s + 3], acc, 0, 0, 0);
    }
    return acc;
}

// out^T(32 features x 32 columns) += tile^T . w, contracting the 32 rows of the LDS tile in the order in which
// the accumulator registers of `w` hold them (row(kk, half) = 8*(kk/4) + 4*half + kk%4).
template <int KS>
__device__ __forceinline__ void accumulate_transposed(v16f& out, const float* tile_col, const v16f& w) {
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
        const float x = tile_col[(8 * (kk >> 2) + (kk & 3)) * KS];
        out = __builtin_amdgcn_mfma_f32_32x32x2f32(x, w[kk], out, 0, 0, 0);
    }
}

// ------------------------------------------------------------------------------------------------------------
// dQ and dbias: a wave owns 32 queries and walks over the keys.
template <int DP, int NW>
__global__ __launch_bounds__(NW * 64) void flash_attn_back_rows_kernel(const AttnBackParams p) {
    constexpr int KS = BackTiling<DP>::KS, NB = DP / 32;
    extern __shared__ __attribute__((aligned(16))) float back_lds[];
    float* lds_k = back_lds;
    float* lds_v = back_lds + p.stage_rows * KS;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 31, half = lane >> 5;
    const int plane = blockIdx.y, L = p.L, d = p.d;
    const int q0 = (blockIdx.x * NW + wave) * 32, q = q0 + j;
    const bool wave_active = q0 < L;
    const int64_t po = static_cast<int64_t>(plane) * L * d;

    float qreg[DP / 2], doreg[DP / 2];
    load_slice<DP>(p.Q + po, q, L, d, half, p.scale * LOG2E, qreg);
    load_slice<DP>(p.dO + po, q, L, d, half, 1.0f, doreg);
    // D_i = sum_d dO_id * O_id: this lane's half of the features, then the other half from lane j + 32
    float D_i = 0.0f;
    {
        float oreg[DP / 2];
        load_slice<DP>(p.O + po, q, L, d, half, 1.0f, oreg);
#pragma unroll
        for (int s = 0; s < DP / 2; ++s) D_i += doreg[s] * oreg[s];
        D_i += lane_xor32(D_i);
    }
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

    const int stage = p.stage_rows;
    for (int c0 = 0; c0 < L; c0 += stage) {
        __syncthreads();
        const int ckeys = L - c0 < stage ? L - c0 : stage;
        const int rows = (ckeys + 31) / 32 * 32;
        stage_pair<DP, NW * 64>(p.K + po, p.V + po, lds_k, lds_v, c0, rows, ckeys, d, tid);
        __syncthreads();
        if (!wave_active) continue;
        for (int kt = 0; kt < rows / 32; ++kt) {
            const int key0 = c0 + kt * 32;
            // ---- probabilities of this lane's query for its 16 keys of the tile
            // bias of this lane's 16 keys, requested before the matrix work (16 bytes at a time)
            float bv[16];
            if (bias_row) {
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
            }
            v16f st = tile_times_slice<DP>(lds_k + (kt * 32 + j) * KS + half * (DP / 2), qreg);
            v16f dp = tile_times_slice<DP>(lds_v + (kt * 32 + j) * KS + half * (DP / 2), doreg);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int key = key0 + 8 * (r >> 2) + 4 * half + (r & 3);
                float s2 = st[r];
                if (bias_row) s2 = __builtin_fmaf(bv[r], LOG2E, s2);
                const float pr = key < row_keys ? __builtin_amdgcn_exp2f(s2 - lse2) : 0.0f;
                st[r] = pr * (dp[r] - D_i);            // dS
            }
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
            if (p.dQ) {
#pragma unroll
                for (int b = 0; b < NB; ++b)
                    accumulate_transposed<KS>(acc_q[b], lds_k + (kt * 32 + 4 * half) * KS + j + 32 * b, st);
            }
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
    constexpr int KS = BackTiling<DP>::KS, NB = DP / 32;
    extern __shared__ __attribute__((aligned(16))) float back_lds[];
    float* lds_q = back_lds;
    float* lds_do = back_lds + p.stage_rows * KS;
    float* lds_lse = lds_do + p.stage_rows * KS;       // LSE * log2(e) of the staged queries (+inf for dead rows)
    float* lds_D = lds_lse + p.stage_rows;             // D of the staged queries
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 31, half = lane >> 5;
    const int plane = blockIdx.y, L = p.L, d = p.d;
    const int k0w = (blockIdx.x * NW + wave) * 32, key = k0w + j;       // this lane's key
    const bool wave_active = k0w < L;
    const int64_t po = static_cast<int64_t>(plane) * L * d;

    float kreg[DP / 2], vreg[DP / 2];
    load_slice<DP>(p.K + po, key, L, d, half, p.scale * LOG2E, kreg);
    load_slice<DP>(p.V + po, key, L, d, half, 1.0f, vreg);
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
        stage_pair<DP, NW * 64>(p.Q + po, p.dO + po, lds_q, lds_do, c0, rows, cq, d, tid);
        // LSE and D = sum_d dO * O of the staged queries: eight threads per row
        for (int idx = tid; idx < rows * 8; idx += NW * 64) {
            const int row = idx >> 3, part = idx & 7;
            float sum = 0.0f;
            if (row < cq) {
                for (int c = part * 4; c < d; c += 32) {
                    const int64_t off = po + static_cast<int64_t>(c0 + row) * d + c;
                    const v4f a = *reinterpret_cast<const v4f*>(p.dO + off), o = *reinterpret_cast<const v4f*>(p.O + off);
                    sum += a[0] * o[0] + a[1] * o[1] + a[2] * o[2] + a[3] * o[3];
                }
            }
            sum += __shfl_xor(sum, 1, 64);
            sum += __shfl_xor(sum, 2, 64);
            sum += __shfl_xor(sum, 4, 64);
            if (part == 0) {
                const float lse = row < cq ? p.LSE[static_cast<int64_t>(plane) * L + c0 + row] : -INFINITY;
                lds_lse[row] = lse > -INFINITY ? lse * LOG2E : INFINITY;
                lds_D[row] = sum;
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
            v16f st = tile_times_slice<DP>(lds_q + (qt * 32 + j) * KS + half * (DP / 2), kreg);
            v16f dp = tile_times_slice<DP>(lds_do + (qt * 32 + j) * KS + half * (DP / 2), vreg);
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
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                if (p.dV) accumulate_transposed<KS>(acc_v[b], lds_do + (qt * 32 + 4 * half) * KS + j + 32 * b, st);
                if (p.dK) accumulate_transposed<KS>(acc_k[b], lds_q + (qt * 32 + 4 * half) * KS + j + 32 * b, ds);
            }
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
    constexpr int NW = 4, KS = BackTiling<DP>::KS, CH = BackTiling<DP>::CH;
    const int l32 = (p.L + 31) / 32 * 32;
    p.stage_rows = l32 < CH ? l32 : CH;
    const dim3 grid((p.L + 32 * NW - 1) / (32 * NW), p.planes), block(NW * 64);
    const size_t lds_rows = static_cast<size_t>(p.stage_rows) * 2 * KS * sizeof(float);
    const size_t lds_cols = lds_rows + static_cast<size_t>(p.stage_rows) * 2 * sizeof(float);
    if (p.dQ || p.dbias) {
        hipLaunchKernelGGL((flash_attn_back_rows_kernel<DP, NW>), grid, block, lds_rows, stream, p);
        const int rc = check_launch("flash_attn_back_rows_kernel");
        if (rc != RC_OK) return rc;
    }
    if (p.dK || p.dV) {
        hipLaunchKernelGGL((flash_attn_back_cols_kernel<DP, NW>), grid, block, lds_cols, stream, p);
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
    stats_record(static_cast<int64_t>(planes) * L, d, L);
    hipStream_t s = static_cast<hipStream_t>(stream);
    return d <= 32 ? launch_back<32>(p, s) : launch_back<64>(p, s);
}
