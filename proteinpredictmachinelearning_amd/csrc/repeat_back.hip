// OP_REPEAT_BACK for gfx950: the sum over the copies a broadcast made, i.e. the gradient of a repeated
// tensor -- in particular of the bias a mul_mat node adds, dbias[n] = sum_m grad[n, m]
// (src/core/ComputeGraph.cpp:724, 742).
//
// Reference behaviour restated here (paths relative to the reference tree):
//   index rule and order of the sum   src/backend/CPUKernels.cpp:2091-2148
//   launcher contract                 src/backend/CUDAKernels.cpp:336-339 (repeat_back4_cuda), 1290-1320
//
// dst[j0,j1,j2,j3] = sum over k0 < r0, k1 < r1, k2 < r2, k3 < r3 of src[j0 + k0*d0, j1 + k1*d1, j2 + k2*d2, j3 + k3*d3]
// with dimension 0 innermost in both tensors.  The reference adds the terms one at a time with k3 running
// fastest; here the same sequence is cut into `slices` consecutive runs that are summed side by side and then
// added in run order, so the result is a fixed function of the shapes (no atomics), equal to the reference's
// up to the rounding of a differently bracketed binary32 sum.
#include "common.hpp"

namespace ppmlhip {
namespace {

struct RepeatBackJob {
    const float* src;
    float* out;                      // dst, or the partial sums [slice][dst element]
    int64_t s0, s1, s2;              // source sizes (dimension 3 follows from the index)
    int64_t d0, d1, d2, d3;          // destination sizes
    int64_t r1, r2, r3;              // copies per dimension (r0 follows from the run bounds)
    int64_t total;                   // d0 * d1 * d2 * d3
    int64_t reps;                    // r0 * r1 * r2 * r3
    int64_t per_slice;               // terms per run
};

// One thread per (destination element, run).  Neighbouring threads hold neighbouring j0, so for every term
// a wave reads one contiguous stretch of the source.
__global__ __launch_bounds__(256) void repeat_back_kernel(const RepeatBackJob jb) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= jb.total) return;
    const int64_t slice = blockIdx.y;
    int64_t t = idx;
    const int64_t j0 = t % jb.d0; t /= jb.d0;
    const int64_t j1 = t % jb.d1; t /= jb.d1;
    const int64_t j2 = t % jb.d2; t /= jb.d2;
    const int64_t j3 = t;
    const int64_t begin = slice * jb.per_slice;
    const int64_t end = begin + jb.per_slice < jb.reps ? begin + jb.per_slice : jb.reps;
    // term number -> (k0, k1, k2, k3), k3 fastest
    int64_t q = begin;
    int64_t k3 = q % jb.r3; q /= jb.r3;
    int64_t k2 = q % jb.r2; q /= jb.r2;
    int64_t k1 = q % jb.r1; q /= jb.r1;
    int64_t k0 = q;
    float sum = 0.0f;
    for (int64_t term = begin; term < end; ++term) {
        const int64_t i0 = j0 + k0 * jb.d0, i1 = j1 + k1 * jb.d1, i2 = j2 + k2 * jb.d2, i3 = j3 + k3 * jb.d3;
        sum += jb.src[((i3 * jb.s2 + i2) * jb.s1 + i1) * jb.s0 + i0];
        if (++k3 == jb.r3) {
            k3 = 0;
            if (++k2 == jb.r2) {
                k2 = 0;
                if (++k1 == jb.r1) { k1 = 0; ++k0; }
            }
        }
    }
    jb.out[slice * jb.total + idx] = sum;
}

__global__ __launch_bounds__(256) void repeat_back_fold_kernel(const float* __restrict__ partial, float* __restrict__ dst,
                                                               int64_t total, int slices) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= total) return;
    float sum = partial[idx];
    for (int s = 1; s < slices; ++s) sum += partial[static_cast<int64_t>(s) * total + idx];
    dst[idx] = sum;
}

}  // namespace
}  // namespace ppmlhip

using namespace ppmlhip;

extern "C" int repeat_back_hip(const float* src, float* dst,
                               int64_t s0, int64_t s1, int64_t s2, int64_t s3,
                               int64_t d0, int64_t d1, int64_t d2, int64_t d3,
                               int64_t r0, int64_t r1, int64_t r2, int64_t r3, ppml_hip_stream_t stream) {
    const bool pos = s0 > 0 && s1 > 0 && s2 > 0 && s3 > 0 && d0 > 0 && d1 > 0 && d2 > 0 && d3 > 0 &&
                     r0 > 0 && r1 > 0 && r2 > 0 && r3 > 0;
    // every term must lie inside the source: (d - 1) + (r - 1) * d < s per dimension, i.e. r <= s / d (a quotient,
    // so that sizes near 2^63 cannot wrap a product past the test)
    const bool inside = pos && r0 <= s0 / d0 && r1 <= s1 / d1 && r2 <= s2 / d2 && r3 <= s3 / d3;
    int64_t total = 0, reps = 0, t01 = 0, t23 = 0, q01 = 0, q23 = 0;
    const bool sized = inside && !__builtin_mul_overflow(d0, d1, &t01) && !__builtin_mul_overflow(d2, d3, &t23) &&
                       !__builtin_mul_overflow(t01, t23, &total) && !__builtin_mul_overflow(r0, r1, &q01) &&
                       !__builtin_mul_overflow(r2, r3, &q23) && !__builtin_mul_overflow(q01, q23, &reps);
    if (!src || !dst || !sized) {
        set_error("repeat_back_hip: bad arguments (src [%lld,%lld,%lld,%lld], dst [%lld,%lld,%lld,%lld], copies [%lld,%lld,%lld,%lld])",
                  (long long)s0, (long long)s1, (long long)s2, (long long)s3, (long long)d0, (long long)d1, (long long)d2,
                  (long long)d3, (long long)r0, (long long)r1, (long long)r2, (long long)r3);
        return RC_BAD_ARGS;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    RepeatBackJob jb{};
    jb.src = src;
    jb.s0 = s0; jb.s1 = s1; jb.s2 = s2;
    jb.d0 = d0; jb.d1 = d1; jb.d2 = d2; jb.d3 = d3;
    jb.r1 = r1; jb.r2 = r2; jb.r3 = r3;
    jb.total = total;
    jb.reps = reps;
    const int64_t blocks = (jb.total + 255) / 256;
    if (blocks > 0x7fffffffLL) { set_error("repeat_back_hip: destination too large"); return RC_BAD_ARGS; }
    // Few destination elements and many copies (a bias gradient: 768 sums of 26368 terms) would leave most of
    // the chip idle: cut the sum into runs until about eight waves per CU have work, at least 32 terms a run.
    int64_t slices = 1;
    const int64_t want_threads = 256LL * 8 * 64;
    if (jb.total < want_threads && jb.reps >= 64) {
        slices = (want_threads + jb.total - 1) / jb.total;
        if (slices > jb.reps / 32) slices = jb.reps / 32;
        if (slices > 65535) slices = 65535;
        if (slices < 1) slices = 1;
    }
    jb.per_slice = (jb.reps + slices - 1) / slices;
    slices = (jb.reps + jb.per_slice - 1) / jb.per_slice;
    float* partial = nullptr;
    if (slices > 1) {
        hipMemPool_t pool = workspace_pool();
        if (!pool || hipMallocFromPoolAsync(reinterpret_cast<void**>(&partial), static_cast<size_t>(slices) * jb.total * 4, pool, s) != hipSuccess) {
            (void)hipGetLastError();
            partial = nullptr;
            slices = 1;                               // no workspace: one run per element, slower and just as right
            jb.per_slice = jb.reps;
        }
    }
    jb.out = partial ? partial : dst;
    hipLaunchKernelGGL(repeat_back_kernel, dim3(static_cast<unsigned>(blocks), static_cast<unsigned>(slices)), dim3(256), 0, s, jb);
    int rc = check_launch("repeat_back_kernel");
    if (partial) {
        if (rc == RC_OK) {
            hipLaunchKernelGGL(repeat_back_fold_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s, partial, dst, jb.total,
                               static_cast<int>(slices));
            rc = check_launch("repeat_back_fold_kernel");
        }
        if (hipFreeAsync(partial, s) != hipSuccess) (void)hipGetLastError();
    }
    return rc;
}
