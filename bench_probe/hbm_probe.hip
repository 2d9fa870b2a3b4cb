// Measurement aid of bench.py, built into its own small library (libppml_probe.so beside this file) and never loaded by the
// backend: a kernel that only moves bytes -- reads `read_bytes` from src and writes `write_bytes` to dst, 16
// bytes per lane, fully coalesced, in one pass of a grid sized like the backend's own kernels.  Timed in the
// same loop as a contraction, it says what a launch that does nothing but that contraction's HBM traffic
// costs on this box (launch latency included), which is the floor the contraction's own time is read against.
#include <hip/hip_runtime.h>
#include <cstdint>

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

template <bool NT>
__global__ __launch_bounds__(256) void stream_kernel(const v4f* __restrict__ src, v4f* __restrict__ dst,
                                                     int64_t read_chunks, int64_t write_chunks, int64_t chunks) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    v4f carry = {0.f, 0.f, 0.f, 0.f};
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < chunks; i += stride) {
        v4f v = {1.f, 2.f, 3.f, 4.f};
        if (i < read_chunks) v = src[i];
        if (i < write_chunks) {
            if (NT) __builtin_nontemporal_store(v, dst + i);
            else dst[i] = v;
        } else {
            carry += v;                                 // the loads beyond the written range stay alive
        }
    }
    if (carry[0] + carry[1] + carry[2] + carry[3] == 1.2345e38f) dst[0] = carry;   // never true for finite data
}

}  // namespace

extern "C" int ppml_probe_stream(const void* src, void* dst, int64_t read_bytes, int64_t write_bytes, int nt,
                                 int work_groups, void* stream) {
    if (!src || !dst || read_bytes < 0 || write_bytes < 0 || (read_bytes % 16) || (write_bytes % 16)) return 1;
    const int64_t rc = read_bytes / 16, wc = write_bytes / 16, chunks = rc > wc ? rc : wc;
    if (chunks == 0) return 0;
    int64_t groups = (chunks + 255) / 256;
    if (work_groups > 0 && groups > work_groups) groups = work_groups;
    if (groups > 0x7fffffff) return 1;
    const dim3 grid(static_cast<unsigned>(groups)), block(256);
    if (nt) hipLaunchKernelGGL(stream_kernel<true>, grid, block, 0, static_cast<hipStream_t>(stream),
                               static_cast<const v4f*>(src), static_cast<v4f*>(dst), rc, wc, chunks);
    else    hipLaunchKernelGGL(stream_kernel<false>, grid, block, 0, static_cast<hipStream_t>(stream),
                               static_cast<const v4f*>(src), static_cast<v4f*>(dst), rc, wc, chunks);
    return hipGetLastError() == hipSuccess ? 0 : 6;
}
