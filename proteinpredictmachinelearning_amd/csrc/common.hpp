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
void stats_record(int64_t M, int64_t K, int64_t N);

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
