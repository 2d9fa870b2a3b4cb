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
// All matrix work is fp32 MFMA (v_mfma_f32_32x32x2_f32), arranged so that nothing has to move
// between lanes:
//
//   scores, transposed:  S^T[key][query] = K_tile (32 keys x d) . Q^T (d x 32 queries)
//       lane (query j = lane % 32, half = lane / 32) ends up with 16 of the 32 keys of ITS query in its
//       accumulator registers -> the softmax row maximum and sum are 16 in-register steps plus one
//       exchange with lane j + 32;
//   output, transposed:  O^T[dd][query] += V^T (d x 32 keys) . P (32 keys x 32 queries)
//       the B operand of step kk is accumulator register kk of the scores -- the key order of the
//       contraction is simply the order in which the score registers hold them (key(kk, half) =
//       8*(kk/4) + 4*half + kk%4), and the V operand is read from LDS in that order;
//       the running rescale factor alpha and the final 1/(l + eps) are per-lane scalars.
//
// The contraction over d likewise runs in the order that lets one 16-byte LDS read feed four MFMA
// steps (slot `half` of step s takes element half*DP/2 + s).
#include "common.hpp"

#include <cmath>

namespace ppmlhip {
namespace {

typedef float v2f __attribute__((ext_vector_type(2)));

template <int DP> struct AttnTiling {
    static constexpr int CH = DP <= 32 ? 256 : 128;   // keys staged in LDS at a time
    static constexpr int KS = DP + 4;                 // row pitch of K in LDS (floats): 16-byte reads, rows 4 banks apart
    static constexpr int VS = DP;                     // row pitch of V
    static constexpr size_t lds_bytes = static_cast<size_t>(CH) * (KS + VS) * sizeof(float);
};

struct AttnParams {
    const float* Q; const float* K; const float* V; const float* bias;
    float* O; float* LSE;
    int planes, L, d;
    int causal;
    float scale, eps;
    int head;            // keys of the reference's first block: min(Bc, keys of the row)
    int stage_rows;      // keys staged in LDS at a time: min(CH, L rounded up to 32)
    int bias_vec;        // bias rows can be read 16 bytes at a time (L % 4 == 0 and an aligned base)
};

__device__ __forceinline__ float lane_xor32(float x) {
    // the value of the lane 32 away (same query, other half of the keys)
    return __shfl_xor(x, 32, 64);
}

template <int DP, int NW>
__global__ __launch_bounds__(NW * 64) void flash_attn_forward_kernel(const AttnParams p) {
    using T = AttnTiling<DP>;
    constexpr int KS = T::KS, VS = T::VS;
    constexpr int NB = DP / 32;                       // 32-row blocks of the transposed output
    extern __shared__ __attribute__((aligned(16))) float attn_lds[];
    float* lds_k = attn_lds;
    float* lds_v = attn_lds + p.stage_rows * KS;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 31, half = lane >> 5;
    const int plane = blockIdx.y;
    const int L = p.L, d = p.d;
    const int q0 = (blockIdx.x * NW + wave) * 32;     // first query of this wave
    const int q = q0 + j;                             // this lane's query
    const bool wave_active = q0 < L;                  // wave-uniform
    const int64_t plane_off = static_cast<int64_t>(plane) * L * d;

    // ---- this lane's slice of its query row: elements half*DP/2 + s, s = 0 .. DP/2-1 (zero past d / past L)
    float qreg[DP / 2];
#pragma unroll
    for (int s = 0; s < DP / 2; s += 4) {
        const int e = half * (DP / 2) + s;
        v4f x = {0.0f, 0.0f, 0.0f, 0.0f};
        if (q < L && e < d) x = *reinterpret_cast<const v4f*>(p.Q + plane_off + static_cast<int64_t>(q) * d + e);
        qreg[s] = x[0]; qreg[s + 1] = x[1]; qreg[s + 2] = x[2]; qreg[s + 3] = x[3];
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
    const float* bias_row = p.bias ? p.bias + (static_cast<int64_t>(plane) * L + (q < L ? q : 0)) * L : nullptr;
    const bool bias_vec = p.bias_vec != 0;

    const int stage = p.stage_rows;
    for (int c0 = 0; c0 < L; c0 += stage) {
        // ---- stage keys c0 .. c0+stage-1 of K and V (zeros past L and past d; whole tiles of 32 only)
        __syncthreads();
        const int ckeys = L - c0 < stage ? L - c0 : stage;
        const int rows = (ckeys + 31) / 32 * 32;
        for (int idx = tid; idx < rows * (DP / 4); idx += NW * 64) {
            const int key = idx / (DP / 4), c = (idx % (DP / 4)) * 4;
            v4f kx = {0.0f, 0.0f, 0.0f, 0.0f}, vx = {0.0f, 0.0f, 0.0f, 0.0f};
            if (key < ckeys && c < d) {
                const int64_t off = plane_off + static_cast<int64_t>(c0 + key) * d + c;
                kx = *reinterpret_cast<const v4f*>(p.K + off);
                vx = *reinterpret_cast<const v4f*>(p.V + off);
            }
            *reinterpret_cast<v4f*>(lds_k + key * KS + c) = kx;
            *reinterpret_cast<v4f*>(lds_v + key * VS + c) = vx;
        }
        __syncthreads();
        if (!wave_active) continue;

        const int tiles_here = (ckeys + 31) / 32;
        for (int kt = 0; kt < tiles_here; ++kt) {
            const int key0 = c0 + kt * 32;             // first key of the tile
            if (key0 >= wave_keys) break;              // causal: nothing left for any query of the wave
            // ---- bias of this lane's 16 keys, requested before the matrix work
            float bv[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) bv[r] = 0.0f;
            if (bias_row && q < L) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int key = key0 + 8 * g + 4 * half;
                    if (bias_vec && key + 3 < L) {
                        const v4f x = *reinterpret_cast<const v4f*>(bias_row + key);
                        bv[4 * g] = x[0]; bv[4 * g + 1] = x[1]; bv[4 * g + 2] = x[2]; bv[4 * g + 3] = x[3];
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; ++i) if (key + i < L) bv[4 * g + i] = bias_row[key + i];
                    }
                }
            }
            // ---- S^T = K_tile . Q^T
            v16f st;
#pragma unroll
            for (int r = 0; r < 16; ++r) st[r] = 0.0f;
            const float* krow = lds_k + (kt * 32 + j) * KS + half * (DP / 2);
#pragma unroll
            for (int s = 0; s < DP / 2; s += 4) {
                const v4f kx = *reinterpret_cast<const v4f*>(krow + s);
                st = __builtin_amdgcn_mfma_f32_32x32x2f32(kx[0], qreg[s], st, 0, 0, 0);
                st = __builtin_amdgcn_mfma_f32_32x32x2f32(kx[1], qreg[s + 1], st, 0, 0, 0);
                st = __builtin_amdgcn_mfma_f32_32x32x2f32(kx[2], qreg[s + 2], st, 0, 0, 0);
                st = __builtin_amdgcn_mfma_f32_32x32x2f32(kx[3], qreg[s + 3], st, 0, 0, 0);
            }
            // ---- scores of this lane's query: scale, bias, masks; tile maximum
            float m_tile = -INFINITY;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int key = key0 + 8 * (r >> 2) + 4 * half + (r & 3);
                float s = st[r] * p.scale;
                s = s + bv[r];
                if (key >= row_keys) s = -INFINITY;
                st[r] = s;
                m_tile = fmaxf(m_tile, s);
                if (key < head_keys) m_head = fmaxf(m_head, s);
            }
            m_tile = fmaxf(m_tile, lane_xor32(m_tile));
            const float m_new = fmaxf(m_run, m_tile);
            const float alpha = (m_run == -INFINITY) ? 0.0f : __expf(m_run - m_new);
            float l_tile = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float pr = (m_new == -INFINITY) ? 0.0f : __expf(st[r] - m_new);
                st[r] = pr;
                l_tile += pr;
            }
            l_tile += lane_xor32(l_tile);
            l_run = alpha * l_run + l_tile;
            m_run = m_new;
            // ---- O^T = alpha * O^T + V^T . P
            const float* vbase = lds_v + (kt * 32 + 4 * half) * VS + j;
#pragma unroll
            for (int b = 0; b < NB; ++b) {
#pragma unroll
                for (int r = 0; r < 16; ++r) acc_o[b][r] *= alpha;
#pragma unroll
                for (int kk = 0; kk < 16; ++kk) {
                    const float vx = vbase[(8 * (kk >> 2) + (kk & 3)) * VS + b * 32];
                    acc_o[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(vx, st[kk], acc_o[b], 0, 0, 0);
                }
            }
        }
    }
    if (!wave_active || q >= L) return;

    // ---- finish the row.  The reference lets a first block of keys that is masked out entirely (all
    // of them -inf) poison the row: its sum becomes NaN and the row is written as O = 0, LSE = -inf
    // (FlashAttn.cpp:96-103, 121-131).  m_head reproduces that outcome.
    m_head = fmaxf(m_head, lane_xor32(m_head));
    const bool live = l_run > 0.0f && m_head > -INFINITY;
    const float inv = live ? 1.0f / (l_run + p.eps) : 0.0f;
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
    if (p.LSE && half == 0) p.LSE[static_cast<int64_t>(plane) * L + q] = live ? m_run + __logf(l_run + p.eps) : -INFINITY;
}

template <int DP, int NW>
int launch_flash(AttnParams p, hipStream_t stream) {
    using T = AttnTiling<DP>;
    auto kernel = &flash_attn_forward_kernel<DP, NW>;
    const int l32 = (p.L + 31) / 32 * 32;
    p.stage_rows = l32 < T::CH ? l32 : T::CH;
    const size_t lds = static_cast<size_t>(p.stage_rows) * (T::KS + T::VS) * sizeof(float);
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

extern "C" int flash_attn_forward_hip(int B, int h, int L, int d, int causal, float scale, float softmax_eps, int Bc,
                                      const float* Q, const float* K, const float* V, const float* bias,
                                      float* O, float* LSE, ppml_hip_stream_t stream) {
    if (!Q || !K || !V || !O || B <= 0 || h <= 0 || L <= 0 || d <= 0) {
        set_error("flash_attn_forward_hip: bad arguments (B=%d h=%d L=%d d=%d)", B, h, L, d);
        return RC_BAD_ARGS;
    }
    if (d > 64 || (d & 3) != 0) {                     // the rule of src/backend/CUDABackend.cpp:457-463
        set_error("flash_attn_forward_hip: head dimension %d not supported (multiple of 4, at most 64)", d);
        return RC_BAD_ARGS;
    }
    const auto misaligned = [](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) != 0; };
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
    p.bias_vec = (bias && (L & 3) == 0 && !misaligned(bias)) ? 1 : 0;
    p.stage_rows = 0;                                 // set per instance
    stats_record(static_cast<int64_t>(planes) * L, d, L);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool few_queries = L <= 128;                // four waves cover the plane
    if (d <= 32) return few_queries ? launch_flash<32, 4>(p, s) : launch_flash<32, 8>(p, s);
    return few_queries ? launch_flash<64, 4>(p, s) : launch_flash<64, 8>(p, s);
}
