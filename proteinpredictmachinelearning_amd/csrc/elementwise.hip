// The element-wise nodes that sit between the matrix multiplications of the reference's graphs, as plain
// streaming kernels: OP_SCALE (the 1/sqrt(D) of the attention logits), OP_UNARY with UNARY_OP_RELU (between the
// two linears of the pair feed-forward), OP_ADD / OP_SUB / OP_MUL / OP_DIV with the reference's flat-modulo
// broadcast (the attention bias), OP_SOFT_MAX over dims[0].  They exist so that a graph built by the reference
// stays on the device between its contractions; where the executor can, it folds them into the neighbouring
// contraction instead (csrc/backend.hip) and these kernels do not run.
//
// All four are bound by HBM: 4 bytes in (8 for the binary ops) and 4 bytes out per element, 16 bytes per lane
// wherever alignment allows.
//
// What they restate of the reference:
//   scale_hip           src/backend/CPUKernels.cpp:1737-1754 (kernel_scale), launcher scale_cuda
//                       (declared src/backend/CUDAKernels.cpp:257, called 992-1004)
//   unary_hip           src/backend/CPUKernels.cpp:2649-2657 (compute_forward_relu), launcher unary_cuda
//                       (declared src/backend/CUDAKernels.cpp:208, called 666-672)
//   bcast_elemwise_hip  src/backend/CPUKernels.cpp:446-596 (kernel_elemwise), launcher bcast_elemwise_cuda
//                       (declared src/backend/CUDAKernels.cpp:114-118, called 678-712)
//   softmax_hip         src/backend/CPUKernels.cpp:1446-1467 (kernel_softmax), launcher softmax_cuda
//                       (declared src/backend/CUDAKernels.cpp:153, called 849-857)
#include "common.hpp"

#include <cmath>

namespace ppmlhip {
namespace {

constexpr int UNARY_OP_RELU = 4;      // include/ppml/ComputeGraph.h:20-25

enum MapOp { MAP_SCALE = 0, MAP_RELU = 1 };

template <int OP>
__device__ __forceinline__ float map1(float v, float s) {
    if (OP == MAP_SCALE) return v * s;
    return v > 0.0f ? v : 0.0f;        // NaN and -0 give +0, as the reference's comparison does
}

// one 16-byte piece per thread; the last, partial piece element by element
template <int OP>
__global__ __launch_bounds__(256) void map_kernel(const float* __restrict__ src, float* __restrict__ dst, int64_t n, float s) {
    const int64_t piece = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int64_t i = piece * 4;
    if (i + 4 <= n) {
        v4f v = *reinterpret_cast<const v4f*>(src + i);
#pragma unroll
        for (int c = 0; c < 4; ++c) v[c] = map1<OP>(v[c], s);
        *reinterpret_cast<v4f*>(dst + i) = v;
    } else {
        for (int64_t j = i; j < n; ++j) dst[j] = map1<OP>(src[j], s);
    }
}

// the same for pointers that are only 4-byte aligned
template <int OP>
__global__ __launch_bounds__(256) void map_scalar_kernel(const float* __restrict__ src, float* __restrict__ dst, int64_t n, float s) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i < n) dst[i] = map1<OP>(src[i], s);
}

template <int EOP>
__device__ __forceinline__ float combine(float a, float b) {
    if (EOP == 0) return a + b;
    if (EOP == 1) return a - b;
    if (EOP == 2) return a * b;
    return a / b;                      // IEEE division: the file is compiled without fast-math
}

// dst[i] = a[i % an] op b[i % bn].  VEC: n, an and bn are multiples of 4 and all three pointers 16-byte aligned, so
// the four elements of a piece are consecutive in every operand.  IDX32: n < 2^32, the remainders are 32-bit.
template <int EOP, bool VEC, bool IDX32>
__global__ __launch_bounds__(256) void bcast_kernel(const float* __restrict__ a, const float* __restrict__ b, float* __restrict__ dst,
                                                    int64_t n, int64_t an, int64_t bn) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int64_t i = VEC ? t * 4 : t;
    if (i >= n) return;
    int64_t ia = i, ib = i;
    if (IDX32) {
        if (an != n) ia = static_cast<uint32_t>(i) % static_cast<uint32_t>(an);
        if (bn != n) ib = static_cast<uint32_t>(i) % static_cast<uint32_t>(bn);
    } else {
        if (an != n) ia = i % an;
        if (bn != n) ib = i % bn;
    }
    if (VEC) {
        const v4f va = *reinterpret_cast<const v4f*>(a + ia);
        const v4f vb = *reinterpret_cast<const v4f*>(b + ib);
        v4f r;
#pragma unroll
        for (int c = 0; c < 4; ++c) r[c] = combine<EOP>(va[c], vb[c]);
        *reinterpret_cast<v4f*>(dst + i) = r;
    } else {
        dst[i] = combine<EOP>(a[ia], b[ib]);
    }
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, 64));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    return v;
}

// One wave per row, the row held in registers between the three passes (maximum, sum of exponentials, quotient):
// it is read once and written once.  PIECES 16-byte pieces (VEC) or single elements per lane.  The reference starts
// its maximum from the first element and moves it with `>` only, so a NaN there stays the maximum; elsewhere a NaN
// is skipped by the maximum and reaches every output through the sum.  Both follow here from fmaxf plus one test.
// HAS_BIAS: the OP_ADD node in front of the softmax folded in (src/modules/Attention.cpp:271-276: scores + bias, then
// softmax): row r of the input plus row r % bias_rows of `bias`, one binary32 addition per element exactly as the node
// would have made it, on the way into the registers -- the sum never goes to memory.
template <int PIECES, bool VEC, bool HAS_BIAS>
__global__ __launch_bounds__(256) void softmax_rows_kernel(const float* __restrict__ in, float* __restrict__ out, int64_t rows, int n,
                                                           const float* __restrict__ bias, int64_t bias_rows) {
    const int lane = threadIdx.x & 63;
    const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float* x = in + row * n;
    const float* b = HAS_BIAS ? bias + (row % bias_rows) * n : nullptr;
    float* y = out + row * n;
    constexpr int W = VEC ? 4 : 1;
    float v[PIECES * W];
    float mx = -INFINITY;
#pragma unroll
    for (int p = 0; p < PIECES; ++p) {
        const int at = (lane + 64 * p) * W;
        if (VEC) {
            v4f t = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
            if (at < n) {
                // (with a bias the inputs need only be 4-byte aligned: see launch_softmax)
                if (HAS_BIAS) t = *reinterpret_cast<const v4f_u*>(x + at);
                else t = *reinterpret_cast<const v4f*>(x + at);
                if (HAS_BIAS) {
                    const v4f tb = *reinterpret_cast<const v4f_u*>(b + at);
#pragma unroll
                    for (int c = 0; c < 4; ++c) t[c] = t[c] + tb[c];
                }
            }
#pragma unroll
            for (int c = 0; c < 4; ++c) v[p * 4 + c] = t[c];
        } else {
            v[p] = at < n ? (HAS_BIAS ? x[at] + b[at] : x[at]) : -INFINITY;
        }
#pragma unroll
        for (int c = 0; c < W; ++c) mx = fmaxf(mx, v[p * W + c]);
    }
    mx = wave_max(mx);
    const float first = __shfl(v[0], 0, 64);
    if (first != first) mx = first;
    float sum = 0.0f;
#pragma unroll
    for (int p = 0; p < PIECES; ++p) {
        const int at = (lane + 64 * p) * W;
#pragma unroll
        for (int c = 0; c < W; ++c) {
            const float e = at + c < n ? expf(v[p * W + c] - mx) : 0.0f;
            v[p * W + c] = e;
            sum += e;
        }
    }
    sum = wave_sum(sum);
    const float inv = 1.0f / (sum + 1e-9f);
#pragma unroll
    for (int p = 0; p < PIECES; ++p) {
        const int at = (lane + 64 * p) * W;
        if (at >= n) continue;
        if (VEC) {
            v4f t;
#pragma unroll
            for (int c = 0; c < 4; ++c) t[c] = v[p * 4 + c] * inv;
            *reinterpret_cast<v4f*>(y + at) = t;
        } else {
            y[at] = v[p] * inv;
        }
    }
}

// Rows too long for a wave's registers: one work-group per row, three passes over memory (the second and third
// come from L2).
template <bool HAS_BIAS>
__global__ __launch_bounds__(256) void softmax_long_rows_kernel(const float* __restrict__ in, float* __restrict__ out, int n,
                                                                const float* __restrict__ bias, int64_t bias_rows) {
    __shared__ float part[4];
    const float* xin = in + static_cast<int64_t>(blockIdx.x) * n;
    const float* b = HAS_BIAS ? bias + (static_cast<int64_t>(blockIdx.x) % bias_rows) * n : nullptr;
    // (the same addition in each of the three passes gives the same value each time)
    const auto x = [&](int i) { return HAS_BIAS ? xin[i] + b[i] : xin[i]; };
    float* y = out + static_cast<int64_t>(blockIdx.x) * n;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    float mx = -INFINITY;
    for (int i = threadIdx.x; i < n; i += 256) mx = fmaxf(mx, x(i));
    mx = wave_max(mx);
    if (lane == 0) part[wave] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
    const float first = x(0);
    if (first != first) mx = first;
    __syncthreads();
    float sum = 0.0f;
    for (int i = threadIdx.x; i < n; i += 256) sum += expf(x(i) - mx);
    sum = wave_sum(sum);
    if (lane == 0) part[wave] = sum;
    __syncthreads();
    sum = (part[0] + part[1]) + (part[2] + part[3]);
    const float inv = 1.0f / (sum + 1e-9f);
    for (int i = threadIdx.x; i < n; i += 256) y[i] = expf(x(i) - mx) * inv;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <int OP>
int launch_map(const char* name, const float* src, float* dst, int64_t n, float s, hipStream_t stream) {
    if (!src || !dst || n < 0) { set_error("%s: bad arguments (n = %lld)", name, (long long)n); return RC_BAD_ARGS; }
    if (n == 0) return RC_OK;
    const bool vec = aligned16(src) && aligned16(dst);
    const int64_t threads = vec ? (n + 3) / 4 : n;
    const int64_t blocks = (threads + 255) / 256;
    if (blocks > 0x7fffffffLL) { set_error("%s: %lld elements are more than one launch takes", name, (long long)n); return RC_BAD_ARGS; }
    if (vec) hipLaunchKernelGGL(map_kernel<OP>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, src, dst, n, s);
    else hipLaunchKernelGGL(map_scalar_kernel<OP>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, src, dst, n, s);
    return check_launch(name);
}

template <int EOP>
int launch_bcast(const float* a, const float* b, float* dst, int64_t n, int64_t an, int64_t bn, hipStream_t stream) {
    const bool vec = (n % 4 == 0) && (an % 4 == 0) && (bn % 4 == 0) && aligned16(a) && aligned16(b) && aligned16(dst);
    const bool idx32 = n < (1LL << 32);
    const int64_t threads = vec ? n / 4 : n;
    const int64_t blocks = (threads + 255) / 256;
    if (blocks > 0x7fffffffLL) { set_error("bcast_elemwise_hip: %lld elements are more than one launch takes", (long long)n); return RC_BAD_ARGS; }
    const dim3 grid(static_cast<unsigned>(blocks)), block(256);
    if (vec && idx32) hipLaunchKernelGGL((bcast_kernel<EOP, true, true>), grid, block, 0, stream, a, b, dst, n, an, bn);
    else if (vec) hipLaunchKernelGGL((bcast_kernel<EOP, true, false>), grid, block, 0, stream, a, b, dst, n, an, bn);
    else if (idx32) hipLaunchKernelGGL((bcast_kernel<EOP, false, true>), grid, block, 0, stream, a, b, dst, n, an, bn);
    else hipLaunchKernelGGL((bcast_kernel<EOP, false, false>), grid, block, 0, stream, a, b, dst, n, an, bn);
    return check_launch("bcast_elemwise_kernel");
}

template <bool VEC, bool HAS_BIAS>
void launch_softmax_rows(int pieces, dim3 grid, hipStream_t stream, const float* in, float* out, int64_t rows, int n,
                         const float* bias, int64_t bias_rows) {
    const dim3 block(256);
    switch (pieces) {
        case 1: hipLaunchKernelGGL((softmax_rows_kernel<1, VEC, HAS_BIAS>), grid, block, 0, stream, in, out, rows, n, bias, bias_rows); break;
        case 2: hipLaunchKernelGGL((softmax_rows_kernel<2, VEC, HAS_BIAS>), grid, block, 0, stream, in, out, rows, n, bias, bias_rows); break;
        case 3: case 4: hipLaunchKernelGGL((softmax_rows_kernel<4, VEC, HAS_BIAS>), grid, block, 0, stream, in, out, rows, n, bias, bias_rows); break;
        default: hipLaunchKernelGGL((softmax_rows_kernel<8, VEC, HAS_BIAS>), grid, block, 0, stream, in, out, rows, n, bias, bias_rows); break;
    }
}

template <bool HAS_BIAS>
int launch_softmax(const char* name, const float* input, const float* bias, float* output, int M, int N, int64_t bias_rows, hipStream_t s) {
    // Which lane holds which element decides the order of the additions in the row's sum, i.e. the last bits of the
    // result.  The folded form has to make the choice the softmax node would have made on the sum the add node would
    // have written -- a tensor of its own, aligned like the output -- so it goes by the output alone and reads its two
    // inputs sixteen bytes at a time wherever they lie.
    const bool vec = (N % 4 == 0) && aligned16(output) && (HAS_BIAS || aligned16(input));
    const int per_lane = vec ? 4 : 1;
    const int pieces = (N + 64 * per_lane - 1) / (64 * per_lane);
    if (pieces <= 8) {
        const dim3 grid(static_cast<unsigned>((static_cast<int64_t>(M) + 3) / 4));
        if (vec) launch_softmax_rows<true, HAS_BIAS>(pieces, grid, s, input, output, M, N, bias, bias_rows);
        else launch_softmax_rows<false, HAS_BIAS>(pieces, grid, s, input, output, M, N, bias, bias_rows);
    } else {
        hipLaunchKernelGGL(softmax_long_rows_kernel<HAS_BIAS>, dim3(static_cast<unsigned>(M)), dim3(256), 0, s, input, output, N, bias, bias_rows);
    }
    return check_launch(name);
}

}  // namespace
}  // namespace ppmlhip

using namespace ppmlhip;

extern "C" int scale_hip(const float* x, float* dst, float scale, int64_t nelements, ppml_hip_stream_t stream) {
    return launch_map<MAP_SCALE>("scale_hip", x, dst, nelements, scale, static_cast<hipStream_t>(stream));
}

extern "C" int unary_hip(const float* src, float* dst, int64_t n, int uop, ppml_hip_stream_t stream) {
    if (uop != UNARY_OP_RELU) {
        set_error("unary_hip: unary op %d is not on this backend's path (UNARY_OP_RELU = %d is)", uop, UNARY_OP_RELU);
        return RC_BAD_ARGS;
    }
    return launch_map<MAP_RELU>("unary_hip", src, dst, n, 0.0f, static_cast<hipStream_t>(stream));
}

extern "C" int bcast_elemwise_hip(const float* a, const float* b, float* dst, int64_t n, int64_t an, int64_t bn, int eop,
                                  ppml_hip_stream_t stream) {
    // an operand shorter than dst repeats along dst's flat order; one that does not divide n is a graph-building
    // error that the reference reads through anyway (CPUKernels.cpp:507-514) -- refused here
    if (!a || !b || !dst || n < 0 || an <= 0 || bn <= 0 || an > n || bn > n || (n % an) != 0 || (n % bn) != 0 || eop < 0 || eop > 3) {
        set_error("bcast_elemwise_hip: bad arguments (n = %lld, an = %lld, bn = %lld, eop = %d)", (long long)n, (long long)an,
                  (long long)bn, eop);
        return RC_BAD_ARGS;
    }
    if (n == 0) return RC_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (eop) {
        case 0: return launch_bcast<0>(a, b, dst, n, an, bn, s);
        case 1: return launch_bcast<1>(a, b, dst, n, an, bn, s);
        case 2: return launch_bcast<2>(a, b, dst, n, an, bn, s);
        default: return launch_bcast<3>(a, b, dst, n, an, bn, s);
    }
}

extern "C" int softmax_hip(const float* input, float* output, int M, int N, ppml_hip_stream_t stream) {
    if (!input || !output || M < 0 || N <= 0) { set_error("softmax_hip: bad arguments (M = %d, N = %d)", M, N); return RC_BAD_ARGS; }
    if (M == 0) return RC_OK;
    return launch_softmax<false>("softmax_kernel", input, nullptr, output, M, N, 1, static_cast<hipStream_t>(stream));
}

extern "C" int softmax_add_hip(const float* input, const float* bias, float* output, int M, int N, int bias_rows,
                               ppml_hip_stream_t stream) {
    if (!input || !bias || !output || M < 0 || N <= 0 || bias_rows <= 0 || (M % bias_rows) != 0) {
        set_error("softmax_add_hip: bad arguments (M = %d, N = %d, bias_rows = %d)", M, N, bias_rows);
        return RC_BAD_ARGS;
    }
    if (M == 0) return RC_OK;
    return launch_softmax<true>("softmax_add_kernel", input, bias, output, M, N, bias_rows, static_cast<hipStream_t>(stream));
}
