// Dimension permutation as a real copy: the twin of the reference's permute_cuda / transpose_cuda
// (declared src/backend/CUDAKernels.cpp:137-143, called from kernel_permute_cuda / kernel_transpose_cuda,
// 1344-1390) with the semantics of CPUBackend::kernel_permute (src/backend/CPUKernels.cpp:1669-1717):
// dimension p of dst is dimension axes[p] of src; both tensors are dense with dims[0] innermost.
// The reference has no strided views: mat_transpose() (ComputeGraphHelper.cpp:375-382), the operand
// shuffles of the backward GEMMs (ComputeGraph.cpp:708-773) and the [L,D,h,B] <-> [D,L,h,B] bridges
// around the fused attention node (ComputeGraphHelper.cpp:450-484) are all this copy.
//
// Pure byte movement, bound by HBM: 4 bytes in and 4 bytes out per element.  Two kernels:
//   * the innermost dimension moves (axes[0] != 0): tiles of 4096 elements go through LDS so that both
//     the reads (along the source's innermost dimension) and the writes (along the destination's) are
//     contiguous runs; the LDS tile has an odd row pitch against bank conflicts;
//   * the innermost dimension stays (axes[0] == 0): rows are copied as they are, 16 bytes per lane
//     when the row length allows.
#include "common.hpp"

namespace ppmlhip {
namespace {

struct PermuteParams {
    const float* src;
    float* dst;
    int64_t sd[4];        // source sizes
    int64_t dd[4];        // destination sizes
    int64_t sstride[4];   // element stride in the source of destination dimension p
    int64_t dstride[4];   // element stride in the destination of destination dimension p
    int64_t planes;       // product of the two destination dimensions that are neither 0 nor c
    int64_t total;
};

// Destination dimension 0 is source dimension a (a != 0); source dimension 0 is destination
// dimension c.  A tile spans T0 indices of destination dimension 0 and TC of destination dimension c
// (T0 * TC = 4096: 64 x 64, or 32 x 128 / 128 x 32 when one of the two dimensions is short, e.g. a head
// dimension of 32); the remaining two destination dimensions are walked by blockIdx.z (and a loop beyond
// 65535 planes).  Element e = tid + 256 k of the tile is read with e running along the source's innermost
// dimension and written with e running along the destination's.
// VEC = 4: both innermost dimensions are multiples of 4 and the pointers 16-byte aligned, so global
// memory is touched 16 bytes per lane on both sides (twice the rate of 4-byte accesses here); the
// LDS tile is accessed element-wise either way.
template <int T0, int TC, int VEC>
__global__ __launch_bounds__(256) void permute_tile_kernel(const PermuteParams p, int c, int r0, int r1) {
    static_assert(T0 * TC == 4096, "16 elements per thread");
    __shared__ float tile[T0][TC + 1];
    const int tid = threadIdx.x;
    const int64_t j0_base = static_cast<int64_t>(blockIdx.x) * T0;  // destination dim 0
    const int64_t jc_base = static_cast<int64_t>(blockIdx.y) * TC;  // destination dim c (source dim 0)
    for (int64_t z = blockIdx.z; z < p.planes; z += gridDim.z) {
        const int64_t jr0 = z % p.dd[r0], jr1 = z / p.dd[r0];
        const int64_t rest_src = jr0 * p.sstride[r0] + jr1 * p.sstride[r1];
        const int64_t rest_dst = jr0 * p.dstride[r0] + jr1 * p.dstride[r1];
#pragma unroll
        for (int k = 0; k < 16 / VEC; ++k) {
            const int e = tid + 256 * k;
            const int col = (e % (TC / VEC)) * VEC, row = e / (TC / VEC);
            const int64_t j0 = j0_base + row, jc = jc_base + col;
            if (j0 < p.dd[0] && jc < p.dd[c]) {                    // VEC = 4: dd[c] % 4 == 0, so all four or none
                const float* src = p.src + rest_src + j0 * p.sstride[0] + jc;
                if (VEC == 4) {
                    const v4f x = *reinterpret_cast<const v4f*>(src);
                    tile[row][col] = x[0]; tile[row][col + 1] = x[1]; tile[row][col + 2] = x[2]; tile[row][col + 3] = x[3];
                } else {
                    tile[row][col] = *src;
                }
            }
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 16 / VEC; ++k) {
            const int e = tid + 256 * k;
            const int row = (e % (T0 / VEC)) * VEC, col = e / (T0 / VEC);
            const int64_t j0 = j0_base + row, jc = jc_base + col;
            if (j0 < p.dd[0] && jc < p.dd[c]) {
                float* dst = p.dst + rest_dst + jc * p.dstride[c] + j0;
                if (VEC == 4) *reinterpret_cast<v4f*>(dst) = v4f{tile[row][col], tile[row + 1][col], tile[row + 2][col], tile[row + 3][col]};
                else *dst = tile[row][col];
            }
        }
        __syncthreads();
    }
}

// The innermost dimension stays: one work-group row of 256 lanes per destination row segment.
template <int VEC>
__global__ __launch_bounds__(256) void permute_rows_kernel(const PermuteParams p) {
    const int64_t n0 = p.dd[0] / VEC;                              // vectors per row
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= p.total / VEC) return;
    const int64_t v = idx % n0;
    int64_t t = idx / n0;
    const int64_t j1 = t % p.dd[1]; t /= p.dd[1];
    const int64_t j2 = t % p.dd[2];
    const int64_t j3 = t / p.dd[2];
    const int64_t off = j1 * p.sstride[1] + j2 * p.sstride[2] + j3 * p.sstride[3] + v * VEC;
    if (VEC == 4) {
        *reinterpret_cast<v4f*>(p.dst + idx * 4) = *reinterpret_cast<const v4f*>(p.src + off);
    } else {
        p.dst[idx] = p.src[off];
    }
}

}  // namespace
}  // namespace ppmlhip

using namespace ppmlhip;

extern "C" int permute_hip(const float* src, float* dst, int64_t total, int ndim,
                           int32_t d0, int32_t d1, int32_t d2, int32_t d3,
                           int64_t s0, int64_t s1, int64_t s2, int64_t s3,
                           int64_t dd0, int64_t dd1, int64_t dd2, int64_t dd3, ppml_hip_stream_t stream) {
    if (!src || !dst || ndim < 1 || ndim > 4 || total < 0) {
        set_error("permute_hip: bad arguments (ndim=%d total=%lld)", ndim, static_cast<long long>(total));
        return RC_BAD_ARGS;
    }
    if (total == 0) return RC_OK;
    int axes[4] = {d0, d1, d2, d3};
    PermuteParams p;
    p.src = src; p.dst = dst; p.total = total; p.planes = 1;
    const int64_t s[4] = {s0, s1, s2, s3}, d[4] = {dd0, dd1, dd2, dd3};
    bool seen[4] = {false, false, false, false};
    for (int i = 0; i < 4; ++i) {
        if (i >= ndim) axes[i] = i;                                 // dimensions past ndim stay in place
        if (axes[i] < 0 || axes[i] >= 4 || (i < ndim && axes[i] >= ndim) || seen[axes[i]]) {
            set_error("permute_hip: axes (%d,%d,%d,%d) are not a permutation of the %d dimensions", d0, d1, d2, d3, ndim);
            return RC_BAD_ARGS;                                     // the reference refuses such a node (CUDAKernels.cpp:1376-1381)
        }
        seen[axes[i]] = true;
        p.sd[i] = i < ndim ? s[i] : 1;
        p.dd[i] = i < ndim ? d[i] : 1;
    }
    int64_t sstr[4] = {1, p.sd[0], p.sd[0] * p.sd[1], p.sd[0] * p.sd[1] * p.sd[2]};
    int64_t count = 1;
    for (int i = 0; i < 4; ++i) {
        if (p.dd[i] != p.sd[axes[i]] || p.dd[i] <= 0) {
            set_error("permute_hip: destination size %lld of dimension %d is not source size %lld of dimension %d",
                      static_cast<long long>(p.dd[i]), i, static_cast<long long>(p.sd[axes[i]]), axes[i]);
            return RC_BAD_ARGS;
        }
        p.sstride[i] = sstr[axes[i]];
        p.dstride[i] = count;
        count *= p.dd[i];
    }
    if (count != total) {
        set_error("permute_hip: total %lld is not the product of the sizes (%lld)", static_cast<long long>(total), static_cast<long long>(count));
        return RC_BAD_ARGS;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (axes[0] == 0) {
        const bool vec = (p.dd[0] & 3) == 0 && ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0;
        const int64_t items = vec ? total / 4 : total;
        const int64_t blocks = (items + 255) / 256;
        if (blocks > 0x7fffffffLL) { set_error("permute_hip: tensor too large"); return RC_BAD_ARGS; }
        if (vec) hipLaunchKernelGGL(permute_rows_kernel<4>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st, p);
        else hipLaunchKernelGGL(permute_rows_kernel<1>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st, p);
        return check_launch("permute_rows_kernel");
    }
    int c = 0;                                                      // destination dimension that is source dimension 0
    for (int i = 0; i < 4; ++i) if (axes[i] == 0) c = i;
    int rest[2], n = 0;
    for (int i = 1; i < 4; ++i) if (i != c) rest[n++] = i;
    p.planes = p.dd[rest[0]] * p.dd[rest[1]];
    const int t0 = p.dd[0] <= 32 ? 32 : (p.dd[c] <= 32 ? 128 : 64), tc = 4096 / t0;
    const int64_t gx = (p.dd[0] + t0 - 1) / t0, gy = (p.dd[c] + tc - 1) / tc, gz = p.planes < 65535 ? p.planes : 65535;
    if (gy > 65535 || gx > 0x7fffffffLL) {
        set_error("permute_hip: grid %lld x %lld exceeds the launch limits", static_cast<long long>(gx), static_cast<long long>(gy));
        return RC_BAD_ARGS;
    }
    const dim3 grid(static_cast<unsigned>(gx), static_cast<unsigned>(gy), static_cast<unsigned>(gz));
    const bool vec = (p.dd[0] & 3) == 0 && (p.dd[c] & 3) == 0 &&
                     ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0;
#define PPML_PERMUTE(T0, TC)                                                                                         \
    do {                                                                                                             \
        if (vec) hipLaunchKernelGGL((permute_tile_kernel<T0, TC, 4>), grid, dim3(256), 0, st, p, c, rest[0], rest[1]); \
        else hipLaunchKernelGGL((permute_tile_kernel<T0, TC, 1>), grid, dim3(256), 0, st, p, c, rest[0], rest[1]);    \
    } while (0)
    if (t0 == 32) PPML_PERMUTE(32, 128);
    else if (t0 == 128) PPML_PERMUTE(128, 32);
    else PPML_PERMUTE(64, 64);
#undef PPML_PERMUTE
    return check_launch("permute_tile_kernel");
}
