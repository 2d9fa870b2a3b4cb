// Shared host/device helpers of the gfx950 mul_mat backend.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <cstdint>
#include <cstdio>
#include <cstdarg>

#include "../../include/ppml_hip.h"

namespace ppmlhip {

constexpr int QK = 32;             // elements per Q8 block (include/ppml/QuantBlocks.h:30)
constexpr int Q8_0_BYTES = 34;     // sizeof(block_q8_0)
constexpr int Q8_1_BYTES = 36;     // sizeof(block_q8_1)

enum Rc { RC_OK = 0, RC_BAD_ARGS = 1, RC_K_NOT_32 = 2, RC_ALLOC = 3, RC_WTYPE = 5, RC_LAUNCH = 6, RC_NO_DEVICE = 7 };

void set_error(const char* fmt, ...);
int  check_launch(const char* what);     // hipGetLastError -> RC_LAUNCH with message

// One launcher call in the MUL_MAT statistics (include/ppml/MulMatStats.h:154-169; the event pair of
// src/cuda/CUDAKernels.cu:1713-1732): counts the call and, outside stream capture, brackets the work
// issued on `stream` during its lifetime with two events.  Costs one relaxed load when statistics are off.
bool stats_enabled();
class StatsScope {
public:
    StatsScope(const char* path, int64_t M, int64_t K, int64_t N, hipStream_t stream);
    ~StatsScope();
    void set_path(const char* path) { path_ = path; }     // a string literal: kept by pointer until the scope ends
    StatsScope(const StatsScope&) = delete;
    StatsScope& operator=(const StatsScope&) = delete;
private:
    const char* path_;
    int64_t M_, K_, N_;
    hipStream_t stream_;
    hipEvent_t e0_ = nullptr, e1_ = nullptr;
    bool on_ = false, timed_ = false;
};
hipMemPool_t workspace_pool();         // the library's stream-ordered pool on the current device, or null
// Device memory for the work a launcher is about to issue on `stream`, valid until that work has run: the stream keeps
// one buffer from the pool between calls (the next taker's work is ordered behind this one's on the same stream, so it
// may have the same memory), which saves an allocation and a release per call -- 10 us on this stack.  Null when none
// is to be had -- always so on a stream under capture.  workspace_give() after the last launch that uses it: it releases
// what was allocated for this call only (the per-thread default stream keeps nothing) and lets the next host thread that
// issues work on the same stream have the buffer (two threads' launches must not interleave on it).
struct Workspace { uint8_t* ptr = nullptr; bool call_owned = false; void* turn = nullptr; };
Workspace workspace_take(size_t bytes, hipStream_t stream);
void workspace_give(const Workspace& ws, hipStream_t stream);
int noalloc_scratch_setup(uint8_t** out);   // address of the no-allocation entry point's static workspace on the current device
int device_cu_count();
void set_q8_path(int path);              // what ppml_hip_q8_last_path() reports for the calling thread

typedef int   v4i  __attribute__((ext_vector_type(4)));
typedef int   v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f  __attribute__((ext_vector_type(4)));
// 4 floats that are only known to be 4-byte aligned (rows of odd length)
typedef float v4f_u __attribute__((ext_vector_type(4), aligned(4)));

// Row that register r of a 32x32 MFMA accumulator holds in lane `lane`; the column is lane % 32.
__device__ __forceinline__ int mfma32_row(int r, int lane) {
    return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
}

// ---- binary32 on the bf16 matrix pipe.  x = x1 + x2 + x3 exactly, each part a bf16 number (8 significant
// bits taken off the top by truncation; the subtractions are exact), so a product of two binary32 numbers
// is the exact sum of nine bf16 x bf16 products; v_mfma_f32_32x32x16_bf16 forms each exactly and adds it
// into a binary32 accumulator.  Six are kept, in this order (smallest first); the other three are below
// 2^-23 of |a||b| together.
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
constexpr int SPLIT_TERMS[6][2] = {{1, 1}, {2, 0}, {0, 2}, {1, 0}, {0, 1}, {0, 0}};   // (part of a, part of b), zero-based

// four consecutive elements -> four bf16 (8 bytes, element order) of each of the three parts
__device__ __forceinline__ void split4(const v4f& v, uint2 (&out)[3]) {
    uint32_t t1[4], t2[4], t3[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const uint32_t b1 = __float_as_uint(v[c]) & 0xffff0000u;
        const float r1 = v[c] - __uint_as_float(b1);              // exact: at most 16 significant bits left
        const uint32_t b2 = __float_as_uint(r1) & 0xffff0000u;
        const float r2 = r1 - __uint_as_float(b2);                // exact: at most 8 significant bits left
        t1[c] = b1; t2[c] = b2; t3[c] = __float_as_uint(r2);
    }
    // the upper halves of two words side by side
    const auto pack = [](uint32_t lo, uint32_t hi) { return __builtin_amdgcn_perm(hi, lo, 0x07060302u); };
    out[0] = uint2{pack(t1[0], t1[1]), pack(t1[2], t1[3])};
    out[1] = uint2{pack(t2[0], t2[1]), pack(t2[2], t2[3])};
    out[2] = uint2{pack(t3[0], t3[1]), pack(t3[2], t3[3])};
}

// What the three parts cannot carry.  The split is exact for every binary32 number whose third part is itself a
// bf16 number; two kinds of operand fall outside that: a non-finite one (x - x1 is NaN, so every product with its
// lower parts is NaN where binary32 arithmetic gives +-inf), and one so small that its lower parts lie below bf16's
// smallest step 2^-133 (they are cut off).  A SplitGuard collects both over the elements a thread splits: the bits
// of the third parts that the packing drops (an OR of the words, looked at once at the end), and the sum of the
// packed third parts (NaN as soon as one of them is -- they are finite numbers below 2^-16 of their operand otherwise,
// so the sum cannot overflow; v_dot2_f32_bf16 adds two of them per instruction).  One vector instruction per element.
// A contraction whose guard fires redoes the affected outputs in plain binary32 arithmetic, one product at a time, k
// ascending: the reference's own loop.
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
struct SplitGuard {
    uint32_t low = 0;
    float sum3 = 0.0f;
    __device__ __forceinline__ bool fired() const { return (low & 0xffffu) != 0 || sum3 != sum3; }
};

__device__ __forceinline__ void split4(const v4f& v, uint2 (&out)[3], SplitGuard& g) {
    uint32_t t1[4], t2[4], t3[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const uint32_t b1 = __float_as_uint(v[c]) & 0xffff0000u;
        const float r1 = v[c] - __uint_as_float(b1);
        const uint32_t b2 = __float_as_uint(r1) & 0xffff0000u;
        const float r2 = r1 - __uint_as_float(b2);
        t1[c] = b1; t2[c] = b2; t3[c] = __float_as_uint(r2);
    }
    const auto pack = [](uint32_t lo, uint32_t hi) { return __builtin_amdgcn_perm(hi, lo, 0x07060302u); };
    out[0] = uint2{pack(t1[0], t1[1]), pack(t1[2], t1[3])};
    out[1] = uint2{pack(t2[0], t2[1]), pack(t2[2], t2[3])};
    out[2] = uint2{pack(t3[0], t3[1]), pack(t3[2], t3[3])};
#if defined(__HIP_DEVICE_COMPILE__)                     // (the host pass of a .hip file knows neither the instruction nor the builtin)
    // The ORs as volatile statements: they stay where they are written.  Left to the scheduler they all sink to the end
    // of a thread's split, with every third part alive until then (the kernels that split in their tile loop are short
    // of registers there: a tenth of a microsecond per launch on the small attention-logit shapes).
    asm volatile("v_or3_b32 %0, %0, %1, %2" : "+v"(g.low) : "v"(t3[0]), "v"(t3[1]));
    asm volatile("v_or3_b32 %0, %0, %1, %2" : "+v"(g.low) : "v"(t3[2]), "v"(t3[3]));
    const v2bf ones = __builtin_bit_cast(v2bf, 0x3f803f80u);
    g.sum3 = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2bf, out[2].x), ones, g.sum3, false);
    g.sum3 = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2bf, out[2].y), ones, g.sum3, false);
#endif
}

// XCD-aware work-group numbering.  Consecutive work-group ids go round-robin over the 8 XCDs, each
// with its own L2.  This maps id -> a logical index such that every XCD walks one contiguous
// eighth of the logical range, so neighbouring tiles (which share operand panels) meet in one L2.
__device__ __forceinline__ int xcd_contiguous_index(int wg, int total) {
    constexpr int XCDS = 8;
    const int per = total / XCDS;            // full rounds
    const int main_part = per * XCDS;
    if (wg >= main_part) return wg;          // ragged tail keeps its id
    return (wg % XCDS) * per + (wg / XCDS);
}

}  // namespace ppmlhip
