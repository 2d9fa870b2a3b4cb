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
// added in a fixed pattern, so the result is a fixed function of the shapes (no atomics), equal to the reference's
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
    int64_t slices;                  // runs (1: `out` is dst itself)
};

// One thread per (run, destination element), the element fastest.  Neighbouring threads hold neighbouring j0, so for
// every term a wave reads one contiguous stretch of the source.  The terms are requested eight at a time and added in their
// order (one load in flight per wave had a bias gradient of 26368 x 768 wait 104 us for 81 MB); the element's place
// moves from term to term by the strides of the four copy counters, no product per term.
__global__ __launch_bounds__(256) void repeat_back_kernel(const RepeatBackJob jb) {
    const int64_t gidx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (gidx >= jb.total * jb.slices) return;
    const int64_t slice = gidx / jb.total;
    const int64_t idx = gidx - slice * jb.total;
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
    // a step of each counter in elements of the source, and what its wrap takes back
    const int64_t st0 = jb.d0, st1 = jb.d1 * jb.s0, st2 = jb.d2 * jb.s1 * jb.s0, st3 = jb.d3 * jb.s2 * jb.s1 * jb.s0;
    const int64_t back3 = jb.r3 * st3, back2 = jb.r2 * st2, back1 = jb.r1 * st1;
    const float* at = jb.src + (((j3 + k3 * jb.d3) * jb.s2 + (j2 + k2 * jb.d2)) * jb.s1 + (j1 + k1 * jb.d1)) * jb.s0 + (j0 + k0 * jb.d0);
    const auto step = [&]() {
        at += st3;
        if (++k3 == jb.r3) {
            k3 = 0; at += st2 - back3;
            if (++k2 == jb.r2) {
                k2 = 0; at += st1 - back2;
                if (++k1 == jb.r1) { k1 = 0; at += st0 - back1; }
            }
        }
    };
    float sum = 0.0f;
    int64_t term = begin;
    for (; term + 8 <= end; term += 8) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) { v[i] = *at; step(); }
#pragma unroll
        for (int i = 0; i < 8; ++i) sum += v[i];
    }
    for (; term < end; ++term) { sum += *at; step(); }
    jb.out[idx * jb.slices + slice] = sum;              // an element's runs side by side, for the wave that adds them
}

// The runs of one destination element, added by one wave: lane l takes runs l, l + 64, ... in their order, then the
// lanes' sums meet in a fixed butterfly -- a fixed function of the shapes, like everything else here.  (One thread
// per element walking its runs one load at a time took longer than the sums themselves: 341 runs for a bias
// gradient of 768 elements.)
__global__ __launch_bounds__(256) void repeat_back_fold_kernel(const float* __restrict__ partial, float* __restrict__ dst,
                                                               int64_t total, int slices) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (idx >= total) return;                           // wave-uniform
    const int lane = threadIdx.x & 63;
    const float* runs = partial + idx * slices;
    float sum = 0.0f;
    for (int s = lane; s < slices; s += 64) sum += runs[s];
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) sum += __shfl_xor(sum, d, 64);
    if (lane == 0) dst[idx] = sum;
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
    // the chip idle: cut the sum into runs until about sixteen waves per CU have work, at least 32 terms a run.
    int64_t slices = 1;
    const int64_t want_threads = 256LL * 16 * 64;
    if (jb.total < want_threads && jb.reps >= 64) {
        slices = (want_threads + jb.total - 1) / jb.total;
        if (slices > jb.reps / 32) slices = jb.reps / 32;
        if (slices > 65535) slices = 65535;
        if (slices < 1) slices = 1;
    }
    jb.per_slice = (jb.reps + slices - 1) / slices;
    slices = (jb.reps + jb.per_slice - 1) / jb.per_slice;
    if (slices > 0x7fffffff / 256 || (jb.total * slices + 255) / 256 > 0x7fffffffLL) { set_error("repeat_back_hip: destination too large"); return RC_BAD_ARGS; }
    float* partial = nullptr;
    Workspace held;
    if (slices > 1) {
        held = workspace_take(static_cast<size_t>(slices) * jb.total * 4, s);
        partial = reinterpret_cast<float*>(held.ptr);
        if (!partial) {
            slices = 1;                               // no workspace: one run per element, slower and just as right
            jb.per_slice = jb.reps;
        }
    }
    jb.out = partial ? partial : dst;
    jb.slices = slices;
    hipLaunchKernelGGL(repeat_back_kernel, dim3(static_cast<unsigned>((jb.total * slices + 255) / 256)), dim3(256), 0, s, jb);
    int rc = check_launch("repeat_back_kernel");
    if (partial) {
        if (rc == RC_OK) {
            hipLaunchKernelGGL(repeat_back_fold_kernel, dim3(static_cast<unsigned>((jb.total + 3) / 4)), dim3(256), 0, s, partial, dst, jb.total,
                               static_cast<int>(slices));
            rc = check_launch("repeat_back_fold_kernel");
        }
        workspace_give(held, s);
    }
    return rc;
}
